"""GPU parity for the sliding-window and attention-sink forms of the decode and prefill
operators against the oracle's fp32 definitions (oracle/paged_ops.py: semantics specified
by this build, PARITY UNPINNED against the reference, whose CPU branches ignore both
arguments).  Covers the three decode kernels (dot-product, matrix-core, block-float-8).
Tolerance atol = rtol = 2e-2 on bf16 outputs."""

import pytest
import torch

import __graft_entry__ as entry
from oracle import bfp8_codec
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


CASES = [
    # users, Hq, Hkv, D, bs, contexts, window
    (4, 32, 8, 128, 64, [5, 64, 200, 700], 128),   # dot-product kernel, window edge inside a tile
    (4, 32, 8, 128, 64, [5, 64, 200, 700], 100),
    (3, 8, 8, 64, 32, [0, 62, 300], 64),           # window = exactly one tile
    (3, 8, 2, 64, 32, [10, 200, 333], 1),          # only the current position
    (2, 64, 8, 128, 64, [1000, 257], 300),         # matrix-core kernel (8 heads per KV head)
    (3, 40, 8, 128, 32, [40, 333, 64], 77),
    (2, 16, 8, 256, 64, [130, 640], 200),          # head size 256
    (2, 8, 8, 128, 64, [90, 500], 4096),           # window longer than every context
]


@pytest.mark.parametrize("users,hq,hkv,d,bs,ctx,window", CASES)
@pytest.mark.parametrize("with_sink", [False, True])
def test_decode_window_and_sink(users, hq, hkv, d, bs, ctx, window, with_sink):
    from tt_xla_amd import workloads

    name = f"decode b{users} h{hq}x{hkv} d{d} bs{bs} ctx{ctx} window{window} sink{with_sink}"
    print(name, flush=True)
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, hq + d + bs + window, users, hq, hkv, d, bs, nb, ctx)
    g = torch.Generator().manual_seed(window)
    sink = (torch.randn(hq, generator=g) * 2).to(torch.bfloat16) if with_sink else None
    dev = wl.to("cuda")
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        dev.q, dev.k_cache, dev.v_cache, dev.page_table, is_causal=True,
        cur_pos_tensor=dev.cache_position, scale=wl.scale, sliding_window_size=window,
        attention_sink=sink.cuda() if with_sink else None)
    want = O.paged_sdpa_decode_windowed(wl.q, wl.k_cache, wl.v_cache, wl.page_table,
                                        wl.cache_position, wl.scale, window, sink)
    _check(name, out.cpu(), want)


@pytest.mark.parametrize("kernel,d", [("mfma", 128), ("mfma16", 128), ("mfma16", 256)])
def test_decode_window_and_sink_matrix_core_kernels(monkeypatch, kernel, d):
    """Window edge inside a tile, sink, short and long users on each matrix-core kernel, with a
    small grid so that wavefronts cross from one windowed segment into the next."""
    from tt_xla_amd import workloads

    monkeypatch.setenv("TTPA_DECODE_KERNEL", kernel)
    monkeypatch.setenv("TTPA_DECODE_WAVES_PER_CU", "1")
    users, hq, hkv, bs, ctx, window = 4, 64, 8, 64, [1990, 30, 1500, 2300], 1000
    name = f"decode [{kernel}] b{users} h{hq}x{hkv} d{d} ctx{ctx} window{window} sink"
    print(name, flush=True)
    nb = sum((c + 1 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged(name, 93, users, hq, hkv, d, bs, nb, ctx)
    g = torch.Generator().manual_seed(3)
    sink = (torch.randn(hq, generator=g) * 2).to(torch.bfloat16)
    dev = wl.to("cuda")
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        dev.q, dev.k_cache, dev.v_cache, dev.page_table, is_causal=True,
        cur_pos_tensor=dev.cache_position, scale=wl.scale, sliding_window_size=window,
        attention_sink=sink.cuda())
    want = O.paged_sdpa_decode_windowed(wl.q, wl.k_cache, wl.v_cache, wl.page_table,
                                        wl.cache_position, wl.scale, window, sink)
    _check(name, out.cpu(), want)


def test_decode_sink_only_and_padded_row():
    from tt_xla_amd import workloads

    wl = workloads.decode_ragged("sink only", 3, 3, 32, 8, 128, 64, 40, [100, 700, 64])
    pos = wl.cache_position.clone()
    pos[1] = -1
    sink = torch.linspace(-4, 4, 32)
    dev = wl.to("cuda")
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        dev.q, dev.k_cache, dev.v_cache, dev.page_table, is_causal=True,
        cur_pos_tensor=pos.cuda(), scale=wl.scale, attention_sink=sink.cuda()).cpu()
    want = O.paged_sdpa_decode_windowed(wl.q, wl.k_cache, wl.v_cache, wl.page_table, pos, wl.scale,
                                        None, sink)
    assert torch.isnan(out[0, 1].float()).all()
    _check("sink only", out[0, [0, 2]], want[0, [0, 2]])
    with pytest.raises(ValueError):
        torch.ops.tt.paged_scaled_dot_product_attention_decode(
            dev.q, dev.k_cache, dev.v_cache, dev.page_table, is_causal=True,
            cur_pos_tensor=dev.cache_position, attention_sink=sink[:5].cuda())
    with pytest.raises(ValueError):
        torch.ops.tt.paged_scaled_dot_product_attention_decode(
            dev.q, dev.k_cache, dev.v_cache, dev.page_table, is_causal=True,
            cur_pos_tensor=dev.cache_position, sliding_window_size=0)


def test_decode_window_on_block_float8_cache():
    """Quantised caches: the comparator is the codec round trip followed by fp32 attention."""
    from tt_xla_amd import custom_ops, workloads

    users, hq, hkv, d, bs, ctx, window = 3, 32, 8, 128, 64, [70, 400, 129], 150
    wl = workloads.decode_ragged("bfp8 window", 9, users, hq, hkv, d, bs, 16, ctx)
    kq, vq = custom_ops.bfp8_pack_cache(wl.k_cache.cuda()), custom_ops.bfp8_pack_cache(wl.v_cache.cuda())
    sink = torch.linspace(-2, 2, hq)
    out = torch.ops.tt.paged_scaled_dot_product_attention_decode(
        wl.q.cuda(), kq, vq, wl.page_table.cuda(), is_causal=True,
        cur_pos_tensor=wl.cache_position.cuda(), scale=wl.scale, sliding_window_size=window,
        attention_sink=sink.cuda())
    k_rt, v_rt = bfp8_codec.roundtrip(wl.k_cache), bfp8_codec.roundtrip(wl.v_cache)
    want = O.paged_sdpa_decode_windowed(wl.q, k_rt, v_rt, wl.page_table, wl.cache_position, wl.scale,
                                        window, sink)
    _check("bfp8 window", out.cpu(), want)


PREFILL = [
    # batch, Hq, Hkv, S, D, window
    (2, 8, 2, 256, 128, 64),
    (1, 8, 8, 192, 64, 50),
    (2, 4, 4, 128, 128, 1),
    (1, 32, 8, 512, 128, 200),
    (1, 4, 2, 128, 256, 33),
    (1, 6, 2, 160, 128, 1000),   # 3 heads per KV head (two row slots per workgroup), window > S
    (1, 6, 2, 320, 128, 70),
]


@pytest.mark.parametrize("b,hq,hkv,s,d,window", PREFILL)
def test_prefill_window(b, hq, hkv, s, d, window):
    g = torch.Generator().manual_seed(s + window)
    q = torch.randn(b, hq, s, d, generator=g).to(torch.bfloat16)
    k = torch.randn(b, hkv, s, d, generator=g).to(torch.bfloat16)
    v = torch.randn(b, hkv, s, d, generator=g).to(torch.bfloat16)
    out = torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=True,
                                                    sliding_window_size=window)
    want = O.sdpa_windowed(q, k, v, sliding_window=window)
    _check(f"prefill b{b} h{hq}x{hkv} s{s} d{d} window{window}", out.cpu(), want)
    with pytest.raises(NotImplementedError):
        torch.ops.tt.scaled_dot_product_attention(q.cuda(), k.cuda(), v.cuda(), is_causal=False,
                                                  sliding_window_size=window)


def test_sliding_ring_decode_flow():
    """Requests decode far past the ring's capacity: ring page tables (rotated sub-rings) +
    window-relative cache positions (tt_xla_amd.sliding_ring, after model_runner.py:1751-1823)
    + the kernels' window mask must reproduce fp32 attention over the newest `window` tokens
    of each request's full history."""
    import numpy as np

    from tt_xla_amd import TTAttentionBackendImpl, TTMetadata
    from tt_xla_amd import sliding_ring as R

    hq, hkv, d, bs, window = 8, 2, 128, 32, 100
    wb = R.sliding_window_blocks(window, bs, max_model_len=4096)  # 8 blocks = 256 positions
    assert wb == 8
    max_reqs = 4
    nb = R.sliding_ring_phys_blocks(wb, max_reqs)
    kv = [torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16, device="cuda") for _ in range(2)]
    impl = TTAttentionBackendImpl(hq, d, d**-0.5, hkv, None, window, "auto")
    gen = torch.Generator().manual_seed(77)
    prompts = {"a": 40, "b": 70}
    total = 340
    q_all = {r: torch.randn(total, hq, d, generator=gen).to(torch.bfloat16) for r in prompts}
    k_all = {r: torch.randn(total, hkv, d, generator=gen).to(torch.bfloat16) for r in prompts}
    v_all = {r: torch.randn(total, hkv, d, generator=gen).to(torch.bfloat16) for r in prompts}
    mapping, free = {}, list(range(max_reqs))
    reqs = list(prompts)
    slots = R.assign_ring_slots(reqs, reqs, mapping, free)

    def expected(r, pos):
        lo = max(0, pos - window + 1)
        k = k_all[r][lo : pos + 1].float().repeat_interleave(hq // hkv, dim=1)
        v = v_all[r][lo : pos + 1].float().repeat_interleave(hq // hkv, dim=1)
        s = torch.einsum("hd,thd->ht", q_all[r][pos].float(), k) * d**-0.5
        return torch.einsum("ht,thd->hd", torch.softmax(s, dim=-1), v)

    # prompt fill: one request per pass, ring table in identity order (context below the window)
    for i, r in enumerate(reqs):
        n = prompts[r]
        start, _ = R.ring_pass_geometry(np.array([n - 1]), bs, wb)
        R.check_ring_fill_supported(start, np.array([0]), np.array([n]))
        table = torch.from_numpy(R.build_sliding_ring_page_table(start, slots[i : i + 1], wb, wb)).to(torch.int32)
        padded = 96
        q = torch.zeros(padded, hq * d, dtype=torch.bfloat16)
        k = torch.zeros(padded, hkv * d, dtype=torch.bfloat16)
        v = torch.zeros(padded, hkv * d, dtype=torch.bfloat16)
        q[:n], k[:n], v[:n] = q_all[r][:n].reshape(n, -1), k_all[r][:n].reshape(n, -1), v_all[r][:n].reshape(n, -1)
        md = TTMetadata(cache_position=None, page_table=table.cuda(), num_users=1,
                        batch_idx=torch.zeros(1, dtype=torch.int32, device="cuda"))
        out = torch.empty(padded, hq * d, dtype=torch.bfloat16, device="cuda")
        impl.forward(None, q.cuda(), k.cuda(), v.cuda(), kv, md, output=out)
        got = out.cpu().view(padded, hq, d)
        for pos in (0, n // 2, n - 1):
            _check(f"ring prefill {r} pos {pos}", got[pos], expected(r, pos))

    # decode both requests together, far past the ring's 256 positions
    pos = np.array([prompts[r] for r in reqs])
    worst = 0.0
    while pos.max() < total:
        start, rel = R.ring_pass_geometry(pos, bs, wb)
        table = torch.from_numpy(R.build_sliding_ring_page_table(start, slots, wb, wb)).to(torch.int32)
        q = torch.stack([q_all[r][p].reshape(-1) for r, p in zip(reqs, pos)])
        k = torch.stack([k_all[r][p].reshape(-1) for r, p in zip(reqs, pos)])
        v = torch.stack([v_all[r][p].reshape(-1) for r, p in zip(reqs, pos)])
        md = TTMetadata(cache_position=torch.from_numpy(rel).to(torch.int32).cuda(),
                        page_table=table.cuda(), num_users=2)
        out = torch.empty(2, hq * d, dtype=torch.bfloat16, device="cuda")
        impl.forward(None, q.cuda(), k.cuda(), v.cuda(), kv, md, output=out)
        if int(pos[0]) % 7 == 0 or int(pos[0]) in (99, 100, 101, 255, 256, 257):
            got = out.cpu().view(2, hq, d)
            for i, r in enumerate(reqs):
                want = expected(r, int(pos[i]))
                worst = max(worst, (got[i].float() - want).abs().max().item())
                torch.testing.assert_close(got[i].float(), want, atol=ATOL, rtol=RTOL)
        pos = pos + 1
    print(f"sliding ring flow: max-abs error {worst:.3e}", flush=True)
