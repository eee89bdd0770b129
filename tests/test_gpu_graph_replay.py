"""GPU tests of the operators under HIP-graph replay, the way bench.py (and a serving loop that
captures its decode forward) runs them: the decode step operator, the one-operator prefill
pass and the two latent operators are captured once and replayed several times with fresh inputs copied into the captured
tensors and eager work between the replays; every replay must equal the eager result on the
same inputs (caches bit for bit, outputs bit for bit: same kernels, same order)."""

import pytest
import torch

import __graft_entry__ as entry

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _pkg():
    entry.ensure_built()
    import tt_xla_amd  # noqa: F401


def _capture(fn):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()  # warm the allocator and the kernels outside capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = fn()
    return graph, out


@pytest.mark.parametrize("bfp8", [False, True])
def test_decode_step_replays(bfp8):
    from tt_xla_amd import custom_ops as ops
    from tt_xla_amd import workloads

    users, hq, hkv, d, bs = 6, 32, 8, 128, 32
    ctx = [5, 64, 200, 700, 20, 1000]  # four more tokens stay inside each user's last block
    nb = sum((c + 4 + bs - 1) // bs for c in ctx) + 3
    wl = workloads.decode_ragged("graph-step", 41, users, hq, hkv, d, bs, nb, ctx).to("cuda")
    pack = ops.bfp8_pack_cache if bfp8 else (lambda t: t.clone())
    k_graph, v_graph = pack(wl.k_cache), pack(wl.v_cache)
    k_eager, v_eager = k_graph.clone(), v_graph.clone()
    q, k_new, v_new, pos = wl.q.clone(), wl.k_new.clone(), wl.v_new.clone(), wl.cache_position.clone()

    def step(kc, vc):
        return torch.ops.tt.paged_update_kv_decode_(q, kc, vc, k_new, v_new, wl.page_table, pos, scale=wl.scale)

    graph, out_graph = _capture(lambda: step(k_graph, v_graph))
    # the capture warm-up and the capture itself leave the graph's caches untouched or written
    # once with the first token; bring both sides to the same state before comparing
    k_graph.copy_(k_eager), v_graph.copy_(v_eager)
    gen = torch.Generator(device="cuda").manual_seed(3)
    for it in range(4):  # four consecutive tokens per user
        q.copy_(torch.randn(q.shape, generator=gen, device="cuda").to(torch.bfloat16))
        k_new.copy_(torch.randn(k_new.shape, generator=gen, device="cuda").to(torch.bfloat16))
        v_new.copy_(torch.randn(v_new.shape, generator=gen, device="cuda").to(torch.bfloat16))
        graph.replay()
        want = step(k_eager, v_eager)  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out_graph, want), f"replay {it}: output differs"
        assert torch.equal(k_graph, k_eager) and torch.equal(v_graph, v_eager), f"replay {it}: caches differ"
        pos += 1


def test_prefill_pass_replays():
    users, s, hq, hkv, d, bs = 2, 192, 16, 4, 128, 32
    g = torch.Generator(device="cuda").manual_seed(9)
    w = s // bs
    nb = users * w + 1
    table = (torch.randperm(nb - 1, generator=g, device="cuda")[: users * w] + 1).view(users, w).to(torch.int32)
    bidx = torch.arange(users, dtype=torch.int32, device="cuda")
    def rnd(*shape):
        return torch.randn(*shape, generator=g, device="cuda").to(torch.bfloat16)
    q, k, v = rnd(users, hq, s, d), rnd(users, hkv, s, d), rnd(users, hkv, s, d)
    kc_g, vc_g = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16, device="cuda"), torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16, device="cuda")
    kc_e, vc_e = kc_g.clone(), vc_g.clone()
    out_g = torch.zeros(users, s, hq, d, dtype=torch.bfloat16, device="cuda")
    out_e = torch.zeros_like(out_g)

    def run(kc, vc, out):
        torch.ops.tt.paged_fill_kv_prefill_out_(q, k, v, kc, vc, table, bidx, out.transpose(1, 2), is_causal=True)

    graph, _ = _capture(lambda: run(kc_g, vc_g, out_g))
    for it in range(3):
        q.copy_(rnd(users, hq, s, d)), k.copy_(rnd(users, hkv, s, d)), v.copy_(rnd(users, hkv, s, d))
        graph.replay()
        run(kc_e, vc_e, out_e)
        torch.cuda.synchronize()
        assert torch.equal(out_g, out_e), f"replay {it}: output differs"
        assert torch.equal(kc_g, kc_e) and torch.equal(vc_g, vc_e), f"replay {it}: caches differ"


@pytest.mark.parametrize("hq", [16, 128])
def test_latent_decode_replays(hq):
    """tt::paged_flash_mla_decode (attention + merge of the partials) captured once: positions, queries
    and cache contents change between the replays."""
    users, dh, dv, bs, width = 5, 576, 512, 64, 20
    g = torch.Generator(device="cuda").manual_seed(17 + hq)
    nb = users * width + 1
    rnd = lambda *shape: torch.randn(*shape, generator=g, device="cuda").to(torch.bfloat16)  # noqa: E731
    q, key = rnd(1, users, hq, dh), rnd(nb, 1, bs, dh)
    table = (torch.randperm(nb - 1, generator=g, device="cuda")[: users * width] + 1).view(users, width).to(torch.int32)
    pos = torch.tensor([0, 63, 500, 1279, 64], dtype=torch.int32, device="cuda")

    def run():
        return torch.ops.tt.paged_flash_mla_decode(q, key, dv, table, None, True, None, pos, None, None)

    graph, out_graph = _capture(run)
    for it in range(3):
        q.copy_(rnd(1, users, hq, dh))
        key[1 + it :: 7].copy_(rnd(*key[1 + it :: 7].shape))
        pos.copy_(torch.tensor([it, 63 + it, 500 - 100 * it, 1279 - it, 64 * (it + 1)], dtype=torch.int32, device="cuda"))
        graph.replay()
        want = run()  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(out_graph, want), f"replay {it}: output differs"


def test_latent_prefill_replays():
    b, hq, s, dh, dv = 2, 16, 160, 576, 512
    g = torch.Generator(device="cuda").manual_seed(23)
    rnd = lambda *shape: torch.randn(*shape, generator=g, device="cuda").to(torch.bfloat16)  # noqa: E731
    q, k = rnd(b, hq, s, dh), rnd(b, 1, s, dh)

    def run():
        return torch.ops.tt.flash_mla_prefill(q, k, dv, None, None, True, dh ** -0.5)

    graph, out_graph = _capture(run)
    for it in range(3):
        q.copy_(rnd(b, hq, s, dh)), k.copy_(rnd(b, 1, s, dh))
        graph.replay()
        want = run()
        torch.cuda.synchronize()
        assert torch.equal(out_graph, want), f"replay {it}: output differs"
