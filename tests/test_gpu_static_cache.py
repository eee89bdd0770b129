"""GPU parity of the non-paged cache operators (tt::update_cache, tt::fill_cache,
tt::scaled_dot_product_attention_decode; reference custom_ops.py:745-950) against the
oracle's restatement: cache writes bit-exact, attention atol = rtol = 2e-2."""

import pytest
import torch

import __graft_entry__ as entry
from oracle import paged_ops as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _bf(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


@pytest.mark.parametrize("b,h,s,d", [(1, 8, 128, 64), (4, 8, 256, 128), (3, 2, 96, 128), (2, 4, 64, 256)])
def test_update_and_fill(b, h, s, d):
    g = torch.Generator().manual_seed(b * s + d)
    cache = _bf(g, b, h, s, d)
    fill1 = _bf(g, b, h, 1, d)
    for p in (0, s // 2 + 1, s - 1):
        pos = torch.tensor([p], dtype=torch.int32)
        got = torch.ops.tt.update_cache(cache.cuda(), fill1.cuda(), pos.cuda(), 0)
        assert torch.equal(got.cpu(), O.update_cache(cache, fill1, pos, 0))
    dev = cache.cuda()
    torch.ops.tt.update_cache_(dev, fill1.cuda(), torch.tensor([3]).cuda(), 0)
    assert torch.equal(dev.cpu(), O.update_cache(cache, fill1, torch.tensor([3]), 0))
    for n in (1, 33, s):
        fill = _bf(g, b, h, n, d)
        got = torch.ops.tt.fill_cache(cache.cuda(), fill.cuda(), 0)
        assert torch.equal(got.cpu(), O.fill_cache(cache, fill, 0))
    # the transposed view a model hands over (tokens-major activations)
    fill = _bf(g, b, 40, h, d).transpose(1, 2)
    dev = cache.cuda()
    torch.ops.tt.fill_cache_(dev, fill.cuda(), 0)
    assert torch.equal(dev.cpu(), O.fill_cache(cache, fill, 0))


def test_update_fill_errors():
    cache = torch.zeros(2, 4, 64, 64, dtype=torch.bfloat16, device="cuda")
    one = torch.zeros(2, 4, 1, 64, dtype=torch.bfloat16, device="cuda")
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(AssertionError):  # batch > 1 needs batch_offset
        torch.ops.tt.update_cache(cache, one, pos)
    with pytest.raises(AssertionError):
        torch.ops.tt.update_cache(cache, one, pos, 1)
    with pytest.raises(AssertionError):
        torch.ops.tt.update_cache(cache, torch.zeros(2, 4, 2, 64, dtype=torch.bfloat16, device="cuda"), pos, 0)
    with pytest.raises(AssertionError):
        torch.ops.tt.fill_cache(cache, torch.zeros(2, 4, 65, 64, dtype=torch.bfloat16, device="cuda"), 0)


@pytest.mark.parametrize("b,hq,hkv,s,d,pos", [
    (1, 8, 8, 128, 64, [100]),
    (4, 32, 8, 256, 128, [0, 63, 64, 255]),
    (3, 16, 2, 512, 128, [511, 17, 300]),     # 8 heads per KV head: matrix-core kernel
    (2, 8, 4, 100, 128, [99, 50]),            # max_seq_len not a multiple of 64
    (2, 8, 8, 128, 256, [5, 127]),
])
def test_static_decode(b, hq, hkv, s, d, pos):
    g = torch.Generator().manual_seed(s + d + hq)
    key, value, q = _bf(g, b, hkv, s, d), _bf(g, b, hkv, s, d), _bf(g, 1, b, hq, d)
    cur = torch.tensor(pos, dtype=torch.int32)
    got = torch.ops.tt.scaled_dot_product_attention_decode(q.cuda(), key.cuda(), value.cuda(), cur.cuda()).cpu()
    want = O.sdpa_decode_static(q, key, value, cur)
    err = (got.float() - want.float()).abs().max().item()
    print(f"static decode b{b} h{hq}x{hkv} s{s} d{d}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)
    table = torch.arange(b, dtype=torch.int32).view(b, 1)
    torch.testing.assert_close(got.float(), O.textbook_decode_fp32(q, key, value, table, cur), atol=2e-2, rtol=2e-2)
    # with a sink (semantics specified by this build, see oracle/paged_ops.py)
    sink = torch.linspace(-3, 3, hq)
    got = torch.ops.tt.scaled_dot_product_attention_decode(q.cuda(), key.cuda(), value.cuda(), cur.cuda(),
                                                           attention_sink=sink.cuda()).cpu()
    want = O.paged_sdpa_decode_windowed(q, key, value, table, cur, None, None, sink)
    torch.testing.assert_close(got.float(), want, atol=2e-2, rtol=2e-2)


@pytest.mark.parametrize("b,hq,d,hkv,s", [
    # the is_causal=False rows of the reference grid (tests/torch/ops/test_custom_ops.py:99-110)
    (1, 12, 128, 12, 32), (1, 12, 128, 12, 128), (8, 12, 128, 12, 128),
    (1, 12, 128, 4, 32), (1, 12, 128, 4, 128), (8, 12, 128, 4, 128),
    (3, 16, 64, 2, 96),   # eight heads per KV head
])
def test_static_decode_with_mask(b, hq, d, hkv, s):
    """attn_mask [B, 1, heads, S] with is_causal=False (reference custom_ops.py:817-842): every
    position, one mask row per query head, against the oracle and against an fp32 loop."""
    g = torch.Generator().manual_seed(s + d + hq + b)
    key, value = _bf(g, b, hkv, s, d), _bf(g, b, hkv, s, d)
    q = (_bf(g, 1, b, hq, d).float() * 0.3).to(torch.bfloat16)
    cur = torch.arange(b, dtype=torch.int32)
    mask = _bf(g, b, 1, hq, s)
    keep = torch.rand(b, 1, hq, s, generator=g) > 0.3
    keep[..., 0] = True
    mask = mask.masked_fill(~keep, float("-inf"))
    got = torch.ops.tt.scaled_dot_product_attention_decode(q.cuda(), key.cuda(), value.cuda(), cur.cuda(),
                                                           mask.cuda(), None, False, 1.0).cpu()
    want = O.sdpa_decode_static(q, key, value, cur, 1.0, mask)
    err = (got.float() - want.float()).abs().max().item()
    print(f"masked static decode b{b} h{hq}x{hkv} s{s} d{d}: max-abs error {err:.3e}", flush=True)
    torch.testing.assert_close(got.float(), want.float(), atol=2e-2, rtol=2e-2)
    grp = hq // hkv
    for u in range(b):
        for h in range(hq):
            w = torch.softmax(q[0, u, h].float() @ key[u, h // grp].float().T + mask[u, 0, h].float(), dim=-1)
            torch.testing.assert_close(got[0, u, h].float(), w @ value[u, h // grp].float(), atol=2e-2, rtol=2e-2)


def test_copy_kv_blocks_round_trip():
    """Block swap (reference model_runner.py:5433-5474): d2h then h2d into other block ids
    reproduces the blocks bit for bit, other blocks stay untouched, and the no-op rules hold."""
    from tt_xla_amd.kv_blocks import copy_kv_blocks

    g = torch.Generator().manual_seed(5)
    dev = {f"layer{i}": [_bf(g, 12, 2, 32, 64).cuda(), _bf(g, 12, 2, 32, 64).cuda()] for i in range(2)}
    dev["fused"] = _bf(g, 12, 2, 32, 64).cuda()
    before = {k: ([t.clone() for t in v] if isinstance(v, list) else v.clone()) for k, v in dev.items()}
    host = {k: ([torch.zeros(6, 2, 32, 64, dtype=torch.bfloat16) for _ in v] if isinstance(v, list)
                else torch.zeros(6, 2, 32, 64, dtype=torch.bfloat16)) for k, v in dev.items()}
    copy_kv_blocks(dev, host, [3, 7, 1], [0, 5, 2], "d2h")
    for k in dev:
        pairs = zip(before[k], host[k]) if isinstance(host[k], list) else [(before[k], host[k])]
        for b, h in pairs:
            assert torch.equal(h[[0, 5, 2]], b[[3, 7, 1]].cpu()) and not h[[1, 3, 4]].any()
    copy_kv_blocks(host, dev, [0, 5, 2], [9, 10, 11], "h2d")
    for k in dev:
        pairs = zip(before[k], dev[k]) if isinstance(dev[k], list) else [(before[k], dev[k])]
        for b, d in pairs:
            assert torch.equal(d[[9, 10, 11]], b[[3, 7, 1]]) and torch.equal(d[:9], b[:9])
    copy_kv_blocks(host, dev, [0], [1, 2], "h2d")  # length mismatch: nothing happens
    copy_kv_blocks({}, dev, [0], [1], "h2d")
    assert torch.equal(dev["fused"][:9], before["fused"][:9])
