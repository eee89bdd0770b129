"""GPU test of ttpa_paged_update_decode_static, the decode-step entry point that allocates
nothing (its split-K partials go to a static array inside the library): called through the C
ABI twice in a row, the second time with a smaller batch, and compared with
ttpa_paged_update_decode on a caller workspace (caches bit for bit, outputs bit for bit: the
same kernels run) and with the CPU oracle (atol = rtol = 2e-2).  Shapes beyond the static
array's size are refused."""

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


def _step_args(dev, out, k_cache, v_cache):
    from tt_xla_amd import custom_ops as ops

    nb, hkv, bs, d, fmt = ops._cache_geometry(k_cache)
    users, hq = dev.q.shape[1], dev.q.shape[2]
    return (
        out.data_ptr(), out.stride(1), out.stride(2), dev.q.data_ptr(), dev.q.stride(1), dev.q.stride(2),
        k_cache.data_ptr(), v_cache.data_ptr(), dev.k_new.data_ptr(), dev.v_new.data_ptr(),
        dev.k_new.stride(1), dev.k_new.stride(2), dev.page_table.data_ptr(), dev.page_table.stride(0),
        dev.cache_position.data_ptr(), 0, users, hq, hkv, d, bs, dev.page_table.shape[1], nb,
        float(dev.scale), fmt, 0, None,
    )


def _run_both(wl):
    """Returns (out, k, v) of the static-scratch entry point and of the workspace one."""
    from tt_xla_amd import _native

    lib = _native.lib()
    dev = wl.to("cuda")
    stream = torch.cuda.current_stream().cuda_stream
    users, hq = dev.q.shape[1], dev.q.shape[2]
    hkv, d = dev.k_cache.shape[1], dev.k_cache.shape[3]

    k_s, v_s, out_s = dev.k_cache.clone(), dev.v_cache.clone(), torch.empty_like(dev.q)
    _native.call("ttpa_paged_update_decode_static", *_step_args(dev, out_s, k_s, v_s), stream)

    k_w, v_w, out_w = dev.k_cache.clone(), dev.v_cache.clone(), torch.empty_like(dev.q)
    nbytes = lib.ttpa_paged_decode_workspace_bytes(users, hq, hkv, d)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    _native.call("ttpa_paged_update_decode", *_step_args(dev, out_w, k_w, v_w), ws.data_ptr(), nbytes, stream)
    torch.cuda.synchronize()
    return (out_s, k_s, v_s), (out_w, k_w, v_w)


def _check(wl):
    (out_s, k_s, v_s), (out_w, k_w, v_w) = _run_both(wl)
    assert torch.equal(k_s, k_w) and torch.equal(v_s, v_w), "caches differ from the workspace entry point's"
    assert torch.equal(out_s.view(torch.int16), out_w.view(torch.int16)), "output differs from the workspace entry point's"
    k_ref = O.paged_update_cache(wl.k_cache, wl.k_new, wl.cache_position, wl.page_table)
    v_ref = O.paged_update_cache(wl.v_cache, wl.v_new, wl.cache_position, wl.page_table)
    assert torch.equal(k_s.cpu(), k_ref) and torch.equal(v_s.cpu(), v_ref), "cache update differs from the oracle"
    ref = O.paged_sdpa_decode(wl.q, k_ref, v_ref, wl.page_table, True, None, wl.cache_position, None, wl.scale)
    err = (out_s.cpu().float() - ref.float()).abs().max().item()
    print(f"{wl.name}: max-abs error vs oracle {err:.3e}", flush=True)
    torch.testing.assert_close(out_s.cpu().float(), ref.float(), atol=ATOL, rtol=RTOL)


def test_two_calls_in_a_row_second_smaller():
    from tt_xla_amd import _native, workloads

    assert _native.lib().ttpa_static_scratch_init() == 0
    big = workloads.decode_ragged("static scratch, 6 users", 11, 6, 32, 8, 128, 64, 80,
                                  [5, 64, 200, 700, 1300, 63])
    small = workloads.decode_ragged("static scratch, 2 users", 12, 2, 32, 8, 128, 64, 20, [130, 301])
    _check(big)
    _check(small)  # the array still holds the first call's table and partials


def test_shape_beyond_the_static_array_is_refused():
    from tt_xla_amd import _native

    lib = _native.lib()
    users, hq, hkv, d = 2048, 128, 8, 256
    assert lib.ttpa_paged_decode_workspace_bytes(users, hq, hkv, d) > lib.ttpa_static_scratch_bytes()
    # rejected on the host, before any pointer is looked at by a kernel
    rc = lib.ttpa_paged_update_decode_static(16, 0, 0, 16, 0, 0, 16, 16, 16, 16, 0, 0, 16, 0, 16, 0, users, hq,
                                             hkv, d, 64, 8, 16, 1.0, 0, 0, None, None)
    assert rc == _native.ERR_WORKSPACE
    assert b"static scratch" in lib.ttpa_last_error()


def test_calls_allocate_no_device_memory_and_replay_from_a_graph():
    """What the entry point exists for: after ttpa_static_scratch_init() and a warm-up call, further
    calls leave the device's free memory unchanged, and a call captured into a graph (where an
    allocation would fail the capture) replays to the eager result."""
    from tt_xla_amd import _native, workloads

    lib = _native.lib()
    assert lib.ttpa_static_scratch_init() == 0
    wl = workloads.decode_ragged("static scratch, no allocation", 13, 5, 32, 8, 128, 64, 64,
                                 [900, 64, 200, 1, 1300])
    dev = wl.to("cuda")
    k, v, out = dev.k_cache.clone(), dev.v_cache.clone(), torch.empty_like(dev.q)
    stream = torch.cuda.current_stream().cuda_stream
    _native.call("ttpa_paged_update_decode_static", *_step_args(dev, out, k, v), stream)  # warm-up
    torch.cuda.synchronize()
    eager = out.clone()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        _native.call("ttpa_paged_update_decode_static", *_step_args(dev, out, k, v), stream)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory moved by {free_before - free_after} bytes over five calls"
    assert torch.equal(out.view(torch.int16), eager.view(torch.int16))

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            _native.call("ttpa_paged_update_decode_static", *_step_args(dev, out, k, v), side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):  # every replay, with eager work in between, against the eager result
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), "a replay differs from the eager call"
