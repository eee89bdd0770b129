#!/usr/bin/env python3
"""Headline benchmark: Llama-3-8B-shaped paged decode on one MI355X.

A step is what one attention layer does for one generated token of every sequence:
K cache update + V cache update + paged decode attention, on synthetic data of the
workload's shape already resident in HBM.  The timed region replays a HIP graph of that
step (captured through the torch.ops.tt operators) on `--rotate` independent copies of
the workload, so consecutive steps never touch the same cache lines.

Prints ONE JSON line: value = algorithmic HBM bytes of a step / time of a step (GB/s),
with tokens/s alongside, the roofline of the dominant kernel (the split-K decode kernel,
timed alone with HIP events) and the CPU oracle timed on this box's host cores.
"""

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "tt-xla_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rotate", type=int, default=3, help="independent workload copies cycled through")
    ap.add_argument("--launch", choices=["graph", "eager"], default="graph")
    ap.add_argument("--workload", choices=["config2", "config4"], default="config2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-users", type=int, default=0, help="users in the CPU sample (0 = auto)")
    return ap.parse_args()


class HipEvents:
    """Raw hipEvent_t pairs; torch's Event type cannot be handed to the C ABI."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def create(self):
        ev = ctypes.c_void_p()
        rc = self.hip.hipEventCreate(ctypes.byref(ev))
        assert rc == 0, f"hipEventCreate -> {rc}"
        return ev

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b)
        assert rc == 0, f"hipEventElapsedTime -> {rc}"
        return ms.value


def make_workload(name, seed, device):
    from tt_xla_amd import workloads

    if name == "config2":
        return workloads.decode_config2(seed=seed, cache_device=device)
    return workloads.decode_config4(seed=seed, cache_device=device)


def step(g):
    import torch

    torch.ops.tt.paged_update_cache_(g.k_cache, g.k_new, g.cache_position, g.page_table)
    torch.ops.tt.paged_update_cache_(g.v_cache, g.v_new, g.cache_position, g.page_table)
    return torch.ops.tt.paged_scaled_dot_product_attention_decode(
        g.q, g.k_cache, g.v_cache, g.page_table, is_causal=True,
        cur_pos_tensor=g.cache_position, scale=g.scale,
    )


def cpu_baseline(args):
    """The CPU oracle (restated reference CPU ops, functional cache clones included) on a
    bounded sample of the same workload: the first `n` users, full-size pool."""
    import torch

    from oracle import paged_ops as O
    from tt_xla_amd import workloads

    cores = os.cpu_count() or 1
    # the box grants 16 cores per GPU whatever os.cpu_count() says
    threads = min(cores, 16)
    torch.set_num_threads(threads)
    wl = make_workload(args.workload, 2, None)
    total_users = wl.q.shape[1]

    def run(n):
        q, kn, vn = wl.q[:, :n], wl.k_new[:, :n], wl.v_new[:, :n]
        pt, pos = wl.page_table[:n], wl.cache_position[:n]
        t0 = time.perf_counter()
        k = O.paged_update_cache(wl.k_cache, kn, pos, pt)
        v = O.paged_update_cache(wl.v_cache, vn, pos, pt)
        O.paged_sdpa_decode(q, k, v, pt, True, None, pos, None, wl.scale)
        return time.perf_counter() - t0

    n = args.cpu_users or min(4, total_users)
    first = run(n)  # warm-up, also sizes the sample
    if not args.cpu_users:
        per_user = max(first / n, 1e-3)
        n = max(1, min(total_users, int(6.0 / per_user)))
    times = [run(n) for _ in range(3)]
    t = statistics.median(times)
    sub = workloads.DecodeWorkload(wl.name, wl.q[:, :n], wl.k_new[:, :n], wl.v_new[:, :n],
                                   wl.k_cache, wl.v_cache, wl.page_table[:n],
                                   wl.cache_position[:n], wl.scale)
    nbytes = sub.decode_bytes() + sub.update_bytes()
    return {
        "value": nbytes / t / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"first {n} of {total_users} users of {wl.name}, full-size cache pool, "
                  f"median of 3 steps after 1 warm-up ({t * 1e3:.0f} ms/step, "
                  f"{n / t:.1f} tokens/s), torch {torch.__version__}",
        "tokens_per_s": n / t,
        "ms_per_step": t * 1e3,
    }


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg in this build "
              "(it shards by KV head / batch with no exchange step); run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import __graft_entry__ as entry

    entry.ensure_built()
    import tt_xla_amd  # noqa: F401
    from tt_xla_amd import _native

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    copies = [make_workload(args.workload, 2 + i, dev).to(dev) for i in range(max(1, args.rotate))]
    wl = copies[0]
    shape = wl.shape
    step_bytes = [c.decode_bytes() + c.update_bytes() for c in copies]
    decode_bytes = [c.decode_bytes() for c in copies]

    # ---- build the launchers -------------------------------------------------------
    if args.launch == "graph":
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for c in copies:  # warm allocator and kernels outside capture
                step(c)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graphs, keep = [], []
        for c in copies:
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                keep.append(step(c))
            graphs.append(gr)
        launchers = [gr.replay for gr in graphs]
    else:
        launchers = [(lambda c=c: step(c)) for c in copies]

    n = len(launchers)
    for i in range(args.warmup):
        launchers[i % n]()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        launchers[i % n]()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    avg_step_bytes = sum(step_bytes[i % n] for i in range(args.steps)) / args.steps
    users = shape["users"]

    # ---- dominant kernel alone: HIP events armed around the split-K decode kernel -------
    ev = HipEvents()
    pairs = []
    k_iters = min(args.steps, 100)
    for i in range(k_iters + 5):
        c = copies[i % n]
        a, b = ev.create(), ev.create()
        _native.call("ttpa_profile_next_attention", a, b)
        step(c)
        if i >= 5:
            pairs.append((a, b, decode_bytes[i % n]))
    torch.cuda.synchronize()
    durs = [ev.elapsed_ms(a, b) for a, b, _ in pairs]
    kern_ms = sum(durs) / len(durs)
    kern_bytes = sum(nb for _, _, nb in pairs) / len(pairs)
    achieved = kern_bytes / (kern_ms * 1e-3) / 1e9

    out = {
        "metric": "paged_decode_attention_hbm_throughput",
        "value": avg_step_bytes / (ms_per_step * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": wl.name,
            "step": "K update + V update + paged decode attention, one layer, one token per sequence",
            "launch": args.launch,
            "rotating_copies": n,
            **shape,
            "mean_context": float(wl.cache_position.float().mean()),
        },
        "tokens_per_s": users / (ms_per_step * 1e-3),
        "pct_of_hbm_peak": 100.0 * avg_step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {
            "kernel": "paged_decode_kernel",
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": None,
            "kernel_us": kern_ms * 1e3,
            "kernel_us_min": min(durs) * 1e3,
            "bytes_per_launch": kern_bytes,
            "timed_launches": len(durs),
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
