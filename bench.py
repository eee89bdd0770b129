#!/usr/bin/env python3
"""Benchmark of the paged KV-cache write + paged attention path on one MI355X.

Default (the headline): Llama-3-8B-shaped paged decode (`--workload config2`).  A step is
what one attention layer does for one generated token of every sequence: K cache update +
V cache update + paged decode attention, on synthetic data of the workload's shape already
resident in HBM.  The timed region replays a HIP graph of that step (captured through the
torch.ops.tt operators) over `--rotate` independent copies of the workload, so consecutive
steps never touch the same cache lines.

Other workloads (same JSON contract):
  config4  Llama-3-70B-shaped decode, batch 128, context 256..32768, fragmented pool
           (its 4 x 512-token chunked-prefill pass is timed separately, see "chunk_pass";
           config5 carries one too: 4 x 512-token chunks over 2048 tokens of block-float-8 cache)
  config5  config2 with a block-float-8 KV cache (dequantised inside the decode kernel)
  config3  causal prefill, 4 x 2048 tokens: K fill + V fill + MFMA attention; value is
           useful TFLOP/s

Prints ONE JSON line.  `roofline` is the dominant kernel alone, timed by a HIP event
pair that its launch carries inside the library; `cpu_baseline` is the CPU oracle timed on this box's host cores on a
bounded sample of the same workload.
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

HBM_PEAK_GBPS = 8000.0      # MI355X published HBM3E bandwidth
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA rate
# HBM bytes per launch of the dominant kernel, from rocprofv3 FETCH_SIZE / WRITE_SIZE counter runs
# of this script scaled by a plain copy of known size (profiles/*_hbm_traffic_*.md).  A counter run
# cannot share a process with the timed run, so the figures are carried here, each with the hash
# of the kernel sources it was measured on (the first 16 hex digits of the SHA-256 over the files
# listed): when the sources have changed since, `roofline.traffic` is null instead of stale.
KERNEL_SOURCES = {
    "paged_decode_mfma16_kernel": ["decode_mfma16_kernel.h", "decode_common.h", "common.h", "decode.hip"],  # the grid rule is in decode.hip
    "paged_decode_latent16_kernel": ["decode_wide.hip", "decode_common.h", "common.h"],
    "paged_decode_latent128_kernel": ["decode_wide.hip", "gen_latent_frag.py", "decode_common.h", "common.h"],
    "latent_prefill_kernel": ["decode_wide.hip", "gen_latent_frag.py", "decode_common.h", "common.h"],
    "prefill_kernel": ["prefill.hip", "gen_prefill_stream.py", "common.h"],
}
MEASURED_TRAFFIC = {
    # workload: (kernel, hash of its sources, HBM bytes per launch: FETCH_SIZE and WRITE_SIZE of the
    # kernel, each scaled by what the same counter reads for a plain copy of known size, mean over
    # the rotating workload copies; the summaries under profiles/ hold the runs)
    "config2": ("paged_decode_mfma16_kernel", "8ba1b647faebb44c", 310422335),
    "config5": ("paged_decode_mfma16_kernel", "8ba1b647faebb44c", 168457090),
    "config4": ("paged_decode_mfma16_kernel", "8ba1b647faebb44c", 3415575936),
    "config3": ("prefill_kernel", "9e5dc9fce6518e7f", 244468287),
    "latent": ("paged_decode_latent16_kernel", "cb2ca9fa245030d1", 654198293),
    "latent128": ("paged_decode_latent128_kernel", "b26a62d6c1d0a108", 739381753),
    "latent-prefill": ("latent_prefill_kernel", "b26a62d6c1d0a108", 332193335),
}
DECODE_KERNEL_NAME = {"config2": "paged_decode_mfma16_kernel", "config4": "paged_decode_mfma16_kernel",
                      "config5": "paged_decode_mfma16_kernel"}
CPU_THREADS_CAP = 16        # host cores a one-GPU box grants, whatever os.cpu_count() says


def kernel_source_hash(kernel):
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES[kernel]:
        with open(os.path.join(ROOT, "tt-xla_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, kernel):
    """The counter-measured HBM bytes per launch for this workload, or None when there is no
    measurement of the kernel as it is built now."""
    rec = MEASURED_TRAFFIC.get(workload)
    if rec is None or rec[0] != kernel or rec[1] != kernel_source_hash(kernel):
        return None
    return rec[2]


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rotate", type=int, default=3, help="independent workload copies cycled through")
    ap.add_argument("--launch", choices=["graph", "eager"], default="graph")
    ap.add_argument("--steps-per-graph", type=int, default=32,
                    help="consecutive steps captured in one graph: a decode forward replays one "
                         "attention step per layer inside one graph, and Llama-3-8B has 32 layers; "
                         "1 = one graph launch per step")
    ap.add_argument("--workload", choices=["config2", "config3", "config4", "config5", "latent", "latent128", "latent-prefill"], default="config2")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="config2 only: leave out the short config3 / config5 runs reported under 'secondary'")
    ap.add_argument("--cpu-users", type=int, default=0, help="users in the CPU sample (0 = auto)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 256 MiB device copies, so that a counter run of this "
                         "command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    return ap.parse_args()


class HipEvents:
    """Raw hipEvent_t pairs; torch's Event type cannot be handed to the C ABI."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]

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


# --------------------------------------------------------------------------- workloads
def make_decode(name, seed, device):
    from tt_xla_amd import workloads

    fn = {"config2": workloads.decode_config2, "config4": workloads.decode_config4,
          "config5": workloads.decode_config5}[name]
    return fn(seed=seed, cache_device=device)


def decode_step(g):
    import torch

    # what the attention backend issues for a decode step: the K / V cache update and the
    # attention as one operator (the update runs inside the decode kernel)
    return torch.ops.tt.paged_update_kv_decode_(
        g.q, g.k_cache, g.v_cache, g.k_new, g.v_new, g.page_table, g.cache_position, scale=g.scale)


def make_prefill_impl(w, kv_cache_dtype="auto"):
    from tt_xla_amd import TTAttentionBackendImpl

    return TTAttentionBackendImpl(w.q_heads, w.head_size, w.head_size**-0.5, w.kv_heads, None, None, kv_cache_dtype)


def time_chunk_pass(w, args, kv_cache_dtype="auto"):
    """A chunked-prefill pass of the backend (fill of the chunk's K / V rows + attention over the cached
    prefix and the chunk), timed as steps and as its attention kernel."""
    import torch

    impl = make_prefill_impl(w, kv_cache_dtype)
    outbuf = torch.empty_like(w.q)
    chunk = [lambda: prefill_step(impl, w, outbuf)]
    cms = time_steps(StepRunner(chunk, args.launch == "graph", args.steps_per_graph), min(args.steps, 50), 5)
    cd = time_dominant_kernel(chunk, 20)
    ck = sum(x for x, _ in cd) / len(cd)
    return {
        "workload": w.name, "ms_per_pass": cms, "attention_kernel_us": ck * 1e3,
        "useful_tflops": w.useful_flops() / (ck * 1e-3) / 1e12,
        "frac_of_bf16_mfma_peak": w.useful_flops() / (ck * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
    }


def prefill_step(impl, w, out):
    """The backend's prefill pass: K fill + V fill + causal attention (dense on the fresh K/V
    for a first chunk, where the backend issues all three as one operator; paged with the
    cached prefix for a continuation chunk)."""
    from tt_xla_amd import TTMetadata

    md = TTMetadata(cache_position=None, page_table=w.page_table, num_users=w.users,
                    batch_idx=w.batch_idx, fill_page_table=w.fill_page_table,
                    chunk_start_idx=w.chunk_start)
    impl.forward(None, w.q, w.k, w.v, [w.k_cache, w.v_cache], md, output=out)
    return out


# --------------------------------------------------------------------------- timing helpers
class StepRunner:
    """Runs steps over the rotating workload copies.  Eager: step i uses copy i % n.  In graph
    mode a graph holds `per_graph` consecutive steps (step j of a graph uses copy j % n; the
    length is chosen so that the last step of a replay and the first of the next use different
    copies), the way the decode forward of a model replays one attention step per layer inside
    one graph; a shorter graph covers the remainder so that run(k) executes exactly k steps.
    sequence(k) lists the copies run(k) goes through."""

    def __init__(self, fns, use_graph, per_graph):
        import torch

        self.fns, self.n, self.use_graph = fns, len(fns), use_graph
        self.per_graph = max(1, per_graph)
        if self.n > 1 and self.per_graph > 1 and (self.per_graph - 1) % self.n == 0:
            self.per_graph += 1
        self.graphs, self.keep = {}, []
        if use_graph:
            # warm-up and capture share one stream
            self.side = torch.cuda.Stream()
            self.side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(self.side):
                for f in fns:  # warm allocator and kernels outside capture
                    f()
            torch.cuda.current_stream().wait_stream(self.side)
            torch.cuda.synchronize()

    def _graph(self, length):
        import torch

        if length not in self.graphs:
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr, stream=self.side):
                for i in range(length):
                    self.keep.append(self.fns[i % self.n]())
            self.graphs[length] = gr
        return self.graphs[length]

    def prepare(self, steps):
        if self.use_graph:
            full, rem = divmod(steps, self.per_graph)
            if full:
                self._graph(self.per_graph)
            if rem:
                self._graph(rem)

    def sequence(self, steps):
        if not self.use_graph:
            return [i % self.n for i in range(steps)]
        full, rem = divmod(steps, self.per_graph)
        return [j % self.n for j in range(self.per_graph)] * full + [j % self.n for j in range(rem)]

    def run(self, steps):
        if not self.use_graph:
            for i in range(steps):
                self.fns[i % self.n]()
            return
        full, rem = divmod(steps, self.per_graph)
        if full:
            gr = self._graph(self.per_graph)
            for _ in range(full):
                gr.replay()
        if rem:
            self._graph(rem).replay()


TIMED_BLOCKS = 7  # the block of `steps` steps is timed this many times; the median is reported


def time_steps_spread(runner, steps, warmup, blocks=TIMED_BLOCKS):
    """(median, min, max) milliseconds per step over `blocks` timed blocks of exactly `steps` steps,
    each bracketed by a device synchronisation on both sides."""
    import torch

    runner.prepare(steps)
    runner.prepare(warmup)
    runner.run(warmup)
    per_step = []
    for _ in range(blocks):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        runner.run(steps)
        torch.cuda.synchronize()
        per_step.append((time.perf_counter() - t0) * 1e3 / steps)
    per_step.sort()
    return per_step[len(per_step) // 2], per_step[0], per_step[-1]


def time_steps(runner, steps, warmup):
    return time_steps_spread(runner, steps, warmup)[0]


def time_dominant_kernel(fns, iters):
    """Eager launches with HIP events armed around the dominant kernel of each call."""
    import torch

    from tt_xla_amd import _native

    ev = HipEvents()
    pairs, n = [], len(fns)
    for i in range(iters + 5):
        a, b = ev.create(), ev.create()
        _native.call("ttpa_profile_next_attention", a, b)
        fns[i % n]()
        if i >= 5:
            pairs.append((a, b, i % n))
    torch.cuda.synchronize()
    return [(ev.elapsed_ms(a, b), which) for a, b, which in pairs]


def time_decode_kernel_direct(copies, iters):
    """The decode kernel alone (the one the step runs: cache update inside), driven through the
    C ABI with preallocated output and workspace: the host enqueues far faster than the GPU executes, so the stream never runs
    dry and the armed event pair, which the kernel's launch carries, reads what a kernel trace reads.  Returns
    [(milliseconds, copy index)]."""
    import torch

    from tt_xla_amd import _native
    from tt_xla_amd import custom_ops as ops

    lib = _native.lib()
    ev = HipEvents()
    stream = torch.cuda.current_stream().cuda_stream
    prepared = []
    for c in copies:
        nb, hkv, bs, d, fmt = ops._cache_geometry(c.k_cache)
        users, hq = c.q.shape[1], c.q.shape[2]
        out = torch.empty_like(c.q)
        nbytes = lib.ttpa_paged_decode_workspace_bytes(users, hq, hkv, d)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=c.q.device)
        prepared.append((c, out, ws, nbytes, (users, hq, hkv, d, bs, c.page_table.shape[1], nb, fmt)))
    pairs, n = [], len(prepared)
    torch.cuda.synchronize()
    for i in range(iters + 10):
        c, out, ws, nbytes, (users, hq, hkv, d, bs, w, nb, fmt) = prepared[i % n]
        a, b = ev.create(), ev.create()
        _native.call("ttpa_profile_next_attention", a, b)
        _native.call(
            "ttpa_paged_update_decode", out.data_ptr(), out.stride(1), out.stride(2),
            c.q.data_ptr(), c.q.stride(1), c.q.stride(2), c.k_cache.data_ptr(), c.v_cache.data_ptr(),
            c.k_new.data_ptr(), c.v_new.data_ptr(), c.k_new.stride(1), c.k_new.stride(2),
            c.page_table.data_ptr(), c.page_table.stride(0), c.cache_position.data_ptr(), 0,
            users, hq, hkv, d, bs, w, nb, float(c.scale), fmt, 0, None, ws.data_ptr(), nbytes, stream)
        if i >= 10:
            pairs.append((a, b, i % n))
    torch.cuda.synchronize()
    return [(ev.elapsed_ms(a, b), which) for a, b, which in pairs]


# --------------------------------------------------------------------------- CPU baselines
def cpu_decode_baseline(args):
    """The CPU oracle (restated reference CPU ops, functional cache clones included) on the
    first `n` users of the workload, full-size pool.  For the block-float-8 workload the CPU
    leg is the codec round trip followed by the same attention."""
    import torch

    from oracle import bfp8_codec
    from oracle import paged_ops as O
    from tt_xla_amd import workloads

    threads = min(os.cpu_count() or 1, CPU_THREADS_CAP)
    torch.set_num_threads(threads)
    if args.workload == "config4":
        wl = workloads.decode_config4(seed=2, num_blocks=16384)
    else:
        wl = make_decode(args.workload, 2, None)
    total_users = wl.q.shape[1]
    k_cache, v_cache = wl.k_cache, wl.v_cache
    note = ""
    if args.workload == "config5":
        t0 = time.perf_counter()
        k_cache = bfp8_codec.roundtrip(k_cache).to(torch.bfloat16)
        v_cache = bfp8_codec.roundtrip(v_cache).to(torch.bfloat16)
        note = f"; codec round trip of both caches (not in the step time) took {time.perf_counter() - t0:.1f} s"

    def run(n):
        q, kn, vn = wl.q[:, :n], wl.k_new[:, :n], wl.v_new[:, :n]
        pt, pos = wl.page_table[:n], wl.cache_position[:n]
        t0 = time.perf_counter()
        k = O.paged_update_cache(k_cache, kn, pos, pt)
        v = O.paged_update_cache(v_cache, vn, pos, pt)
        O.paged_sdpa_decode(q, k, v, pt, True, None, pos, None, wl.scale)
        return time.perf_counter() - t0

    n = args.cpu_users or min(2, total_users)
    first = run(n)
    if not args.cpu_users:
        n = max(1, min(total_users, 16 if args.workload == "config4" else total_users,
                       int(6.0 / max(first / n, 1e-3))))
    times = [run(n) for _ in range(3)]
    t = statistics.median(times)
    sub = workloads.DecodeWorkload(wl.name, wl.q[:, :n], wl.k_new[:, :n], wl.v_new[:, :n],
                                   wl.k_cache, wl.v_cache, wl.page_table[:n],
                                   wl.cache_position[:n], wl.scale)
    e_kv = 17.0 / 16.0 if args.workload == "config5" else 2.0
    nbytes = sub.decode_bytes(e_kv) + sub.update_bytes()
    return {
        "value": nbytes / t / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"first {n} of {total_users} users of {wl.name}, full-size cache pool, median of 3 "
                  f"steps after 1 warm-up ({t * 1e3:.0f} ms/step, {n / t:.1f} tokens/s), "
                  f"torch {torch.__version__}{note}",
        "tokens_per_s": n / t, "ms_per_step": t * 1e3,
    }


def cpu_prefill_baseline(args):
    import torch

    from oracle import paged_ops as O
    from tt_xla_amd import workloads

    threads = min(os.cpu_count() or 1, CPU_THREADS_CAP)
    torch.set_num_threads(threads)
    w = workloads.prefill_config3()
    n, s = 1, w.seq
    q = w.q[: n * s].view(n, s, w.q_heads, w.head_size).transpose(1, 2)
    k = w.k[: n * s].view(n, s, w.kv_heads, w.head_size).transpose(1, 2)
    v = w.v[: n * s].view(n, s, w.kv_heads, w.head_size).transpose(1, 2)
    bidx = w.batch_idx[:n]

    def run():
        t0 = time.perf_counter()
        kc = O.paged_fill_cache_batched(w.k_cache, k, w.fill_page_table, bidx)
        vc = O.paged_fill_cache_batched(w.v_cache, v, w.fill_page_table, bidx)
        O.sdpa(q, k, v, None, True, w.head_size**-0.5)
        del kc, vc
        return time.perf_counter() - t0

    run()
    t = statistics.median([run() for _ in range(3)])
    flops = w.useful_flops() * n / w.users
    return {
        "value": flops / t / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"first {n} of {w.users} prompts of {w.name} (fill K, fill V with functional cache "
                  f"clones, causal attention), median of 3 after 1 warm-up ({t * 1e3:.0f} ms), "
                  f"torch {torch.__version__}",
        "ms_per_step": t * 1e3,
    }


# --------------------------------------------------------------------------- runs
def run_decode(args):
    import torch

    from tt_xla_amd import custom_ops as ops

    dev = "cuda:0"
    copies = [make_decode(args.workload, 2 + i, dev).to(dev) for i in range(max(1, args.rotate))]
    e_kv, dtype = 2.0, "bf16"
    if args.workload == "config5":
        for c in copies:  # caches become block-float-8 (uint8) tensors
            c.k_cache = ops.bfp8_pack_cache(c.k_cache)
            c.v_cache = ops.bfp8_pack_cache(c.v_cache)
        e_kv, dtype = 17.0 / 16.0, "bfp8 cache, bf16 activations, f32 accumulate"
        torch.cuda.empty_cache()
    wl = copies[0]
    nb, hkv, _, d = wl.k_cache.shape
    shape = dict(users=wl.q.shape[1], q_heads=wl.q.shape[2], kv_heads=hkv, head_size=d,
                 block_size=64, num_blocks=nb, table_width=wl.page_table.shape[1])
    dec_bytes = [c.decode_bytes(e_kv) for c in copies]
    step_bytes = [b + c.update_bytes() for b, c in zip(dec_bytes, copies)]
    fns = [(lambda c=c: decode_step(c)) for c in copies]
    runner = StepRunner(fns, args.launch == "graph", args.steps_per_graph)
    ms, ms_min, ms_max = time_steps_spread(runner, args.steps, args.warmup)
    n = len(copies)
    avg_step_bytes = sum(step_bytes[i] for i in runner.sequence(args.steps)) / args.steps
    durs = time_decode_kernel_direct(copies, min(args.steps, 100))
    kern_ms = sum(d for d, _ in durs) / len(durs)
    kern_bytes = sum(step_bytes[w] for _, w in durs) / len(durs)  # the kernel also writes the new token
    achieved = kern_bytes / (kern_ms * 1e-3) / 1e9
    out = {
        "metric": "paged_decode_attention_hbm_throughput",
        "value": avg_step_bytes / (ms * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms,
        "ms_per_step_min": ms_min, "ms_per_step_max": ms_max, "timed_blocks": TIMED_BLOCKS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {
            "workload": wl.name,
            "step": "K + V cache update and paged decode attention (one operator: the update runs inside the decode kernel) + merge of the split-K partials, one layer, one token per sequence",
            "launch": args.launch, "steps_per_graph": runner.per_graph if args.launch == "graph" else None,
            "rotating_copies": n, **shape,
            "mean_context": float(wl.cache_position.float().mean()),
        },
        "tokens_per_s": shape["users"] / (ms * 1e-3),
        "pct_of_hbm_peak": 100.0 * avg_step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {
            "kernel": DECODE_KERNEL_NAME[args.workload],
            "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": measured_traffic(args.workload, DECODE_KERNEL_NAME[args.workload]),
            "kernel_source_hash": kernel_source_hash(DECODE_KERNEL_NAME[args.workload]),
            "kernel_us": kern_ms * 1e3, "kernel_us_min": min(d for d, _ in durs) * 1e3,
            "bytes_per_launch": kern_bytes, "timed_launches": len(durs),
        },
    }
    if args.workload == "config4":
        from tt_xla_amd import workloads

        out["chunk_pass"] = time_chunk_pass(workloads.prefill_config4_chunks(device=dev).to(dev), args)
    if args.workload == "config5":
        from tt_xla_amd import workloads

        # the chunked-prefill pass over the same kind of cache: 4 x 512-token chunks on 2048 cached tokens
        w = workloads.prefill_workload("config5-chunks-b4x512-start2048-h32x8-d128-bs64-bfp8", 55, 4, 512, 32, 8,
                                       128, 64, 2048, dev).to(dev)
        w.k_cache, w.v_cache = ops.bfp8_pack_cache(w.k_cache), ops.bfp8_pack_cache(w.v_cache)
        out["chunk_pass"] = time_chunk_pass(w, args, "uint8")
    return out


def run_latent(args, hq=16):
    """Latent (MLA) decode at the shape one rank of a latent-attention model serves: 16 query heads
    over one latent KV head of 576 = 512 + 64 features, V = its 512 leading features; 128 users,
    contexts uniform in [512, 8192], block 64.  The step is tt::paged_flash_mla_decode (attention +
    merge of the split-K partials); the cache write of the step is the plain tt::paged_update_cache
    on the latent cache and is not part of it.  hq = 128 is the layer with all of its heads on one
    GPU: 242 flop per byte of the cache, so the matrix pipes bound it and not the memory; the
    figure stays in bytes per second so that the two shapes read on one scale."""
    import torch

    users, dh, dv, bs, lo, hi = 128, 576, 512, 64, 512, 8192
    dev = "cuda:0"
    copies = []
    for i in range(max(1, min(args.rotate, 2))):
        g = torch.Generator().manual_seed(11 + i)
        ctx = torch.randint(lo, hi + 1, (users,), generator=g)
        w = (hi + bs) // bs
        nb = users * w + 1
        key = torch.randn(nb, 1, bs, dh, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
        table = (torch.randperm(nb - 1, generator=g)[: users * w] + 1).view(users, w).to(torch.int32).to(dev)
        q = torch.randn(1, users, hq, dh, generator=g, dtype=torch.float32).to(torch.bfloat16).to(dev)
        copies.append((q, key, table, ctx.to(torch.int32).to(dev), int((ctx + 1).sum())))
    fns = [(lambda c=c: torch.ops.tt.paged_flash_mla_decode(c[0], c[1], dv, c[2], None, True, None, c[3], None, None))
           for c in copies]
    nbytes = [c[4] * dh * 2 + users * hq * (dh + dv) * 2 + users * (c[2].shape[1] * 4 + 4) for c in copies]
    runner = StepRunner(fns, args.launch == "graph", args.steps_per_graph)
    steps = min(args.steps, 100)
    ms, ms_min, ms_max = time_steps_spread(runner, steps, min(args.warmup, 10))
    avg_bytes = sum(nbytes[i] for i in runner.sequence(steps)) / steps
    durs = time_dominant_kernel(fns, min(steps, 50))
    kern_ms = sum(d for d, _ in durs) / len(durs)
    kern_bytes = sum(nbytes[w] for _, w in durs) / len(durs)
    achieved = kern_bytes / (kern_ms * 1e-3) / 1e9
    kernel = "paged_decode_latent16_kernel" if hq <= 16 else "paged_decode_latent128_kernel"
    flops = 2.0 * kern_bytes / (dh * 2) * hq * (dh + dv)
    return {
        "metric": "paged_decode_attention_hbm_throughput",
        "value": avg_bytes / (ms * 1e-3) / 1e9, "unit": "GB/s",
        "n_gpus": 1, "steps": steps, "warmup": min(args.warmup, 10), "ms_per_step": ms,
        "ms_per_step_min": ms_min, "ms_per_step_max": ms_max, "timed_blocks": TIMED_BLOCKS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"latent-decode-b{users}-h{hq}x1-d{dh}/{dv}-bs{bs}-ctx{lo}..{hi}",
            "step": "paged latent decode attention + merge of the split-K partials, one layer, one token per sequence",
            "launch": args.launch, "steps_per_graph": runner.per_graph if args.launch == "graph" else None,
            "rotating_copies": len(copies), "users": users, "q_heads": hq, "kv_heads": 1, "head_size": dh,
            "head_dim_v": dv, "block_size": bs,
        },
        "tokens_per_s": users / (ms * 1e-3),
        "pct_of_hbm_peak": 100.0 * avg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {
            "kernel": kernel, "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS, "traffic": measured_traffic("latent" if hq <= 16 else "latent128", kernel),
            "kernel_source_hash": kernel_source_hash(kernel),
            "kernel_us": kern_ms * 1e3, "kernel_us_min": min(d for d, _ in durs) * 1e3,
            "bytes_per_launch": kern_bytes, "timed_launches": len(durs),
            "tflops": flops / (kern_ms * 1e-3) / 1e12,
            "frac_of_bf16_mfma_peak": flops / (kern_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
        },
    }


def run_latent_prefill(args):
    """tt::flash_mla_prefill at the latent serving shape: 4 prompts of 2048 tokens, 16 query heads
    over one latent head of 576 features, V = its 512 leading ones, causal.  Useful flops:
    2 (576 + 512) per (row, key <= row) pair."""
    import torch

    b, hq, s, dh, dv = 4, 16, 2048, 576, 512
    dev = "cuda:0"
    copies = []
    for i in range(max(1, min(args.rotate, 2))):
        g = torch.Generator().manual_seed(21 + i)
        q = (torch.randn(b, hq, s, dh, generator=g) * 0.15).to(torch.bfloat16).to(dev)
        k = torch.randn(b, 1, s, dh, generator=g).to(torch.bfloat16).to(dev)
        copies.append((q, k))
    fns = [(lambda c=c: torch.ops.tt.flash_mla_prefill(c[0], c[1], dv, None, None, True, dh ** -0.5)) for c in copies]
    runner = StepRunner(fns, args.launch == "graph", args.steps_per_graph)
    steps = min(args.steps, 100)
    ms, ms_min, ms_max = time_steps_spread(runner, steps, min(args.warmup, 10))
    flops = 2.0 * b * hq * (s * (s + 1) / 2) * (dh + dv)
    durs = time_dominant_kernel(fns, min(steps, 50))
    kern_ms = sum(d for d, _ in durs) / len(durs)
    achieved = flops / (kern_ms * 1e-3) / 1e12
    return {
        "metric": "latent_prefill_attention_useful_tflops",
        "value": flops / (ms * 1e-3) / 1e12, "unit": "TFLOP/s",
        "n_gpus": 1, "steps": steps, "warmup": min(args.warmup, 10), "ms_per_step": ms,
        "ms_per_step_min": ms_min, "ms_per_step_max": ms_max, "timed_blocks": TIMED_BLOCKS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"latent-prefill-b{b}x{s}-h{hq}x1-d{dh}/{dv}",
            "step": "causal latent prefill attention over freshly built latent K (V = its leading features), one launch",
            "launch": args.launch, "steps_per_graph": runner.per_graph if args.launch == "graph" else None,
            "rotating_copies": len(copies), "users": b, "tokens_per_user": s, "q_heads": hq, "kv_heads": 1,
            "head_size": dh, "head_dim_v": dv,
        },
        "tokens_per_s": b * s / (ms * 1e-3),
        "roofline": {
            "kernel": "latent_prefill_kernel", "bound": "mfma", "achieved": achieved,
            "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / MFMA_BF16_PEAK_TFLOPS,
            "traffic": measured_traffic("latent-prefill", "latent_prefill_kernel"),
            "kernel_source_hash": kernel_source_hash("latent_prefill_kernel"),
            "kernel_us": kern_ms * 1e3, "kernel_us_min": min(d for d, _ in durs) * 1e3,
            "flops_per_launch": flops, "timed_launches": len(durs),
        },
    }


def run_prefill(args):
    import torch

    from tt_xla_amd import workloads

    dev = "cuda:0"
    copies = [workloads.prefill_config3(seed=3 + i, device=dev).to(dev) for i in range(max(1, args.rotate))]
    impls = [make_prefill_impl(w) for w in copies]
    outs = [torch.empty_like(w.q) for w in copies]
    fns = [(lambda i=i: prefill_step(impls[i], copies[i], outs[i])) for i in range(len(copies))]
    runner = StepRunner(fns, args.launch == "graph", args.steps_per_graph)
    steps = min(args.steps, 100)
    ms, ms_min, ms_max = time_steps_spread(runner, steps, min(args.warmup, 10))
    w = copies[0]
    flops = w.useful_flops()
    durs = time_dominant_kernel(fns, min(steps, 50))
    kern_ms = sum(d for d, _ in durs) / len(durs)
    achieved = flops / (kern_ms * 1e-3) / 1e12
    return {
        "metric": "paged_prefill_attention_useful_tflops",
        "value": flops / (ms * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": steps, "warmup": min(args.warmup, 10), "ms_per_step": ms,
        "ms_per_step_min": ms_min, "ms_per_step_max": ms_max, "timed_blocks": TIMED_BLOCKS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": w.name,
            "step": "K fill + V fill through the fill page table + causal attention on the fresh K/V "
                    "(one operator, one launch: extra workgroups of the attention kernel copy the rows)",
            "launch": args.launch, "steps_per_graph": runner.per_graph if args.launch == "graph" else None,
            "rotating_copies": len(copies), "users": w.users,
            "tokens_per_user": w.seq, "q_heads": w.q_heads, "kv_heads": w.kv_heads,
            "head_size": w.head_size, "block_size": 64,
        },
        "tokens_per_s": w.users * w.seq / (ms * 1e-3),
        "fill_bytes_per_step": w.fill_bytes(),
        "roofline": {
            "kernel": "prefill_kernel", "bound": "mfma", "achieved": achieved,
            "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved / MFMA_BF16_PEAK_TFLOPS, "traffic": measured_traffic("config3", "prefill_kernel"),
            "kernel_source_hash": kernel_source_hash("prefill_kernel"),
            "kernel_us": kern_ms * 1e3, "kernel_us_min": min(d for d, _ in durs) * 1e3,
            "flops_per_launch": flops, "timed_launches": len(durs),
            "note": "useful (causal) FLOPs only; the dense 4*B*Hq*S^2*D figure is twice this; the launch "
                    "also carries the step's K / V cache fill (fill_bytes_per_step of traffic)",
        },
    }


def run_workload(args):
    if args.workload == "config3":
        return run_prefill(args)
    if args.workload == "latent":
        return run_latent(args)
    if args.workload == "latent128":
        return run_latent(args, hq=128)
    if args.workload == "latent-prefill":
        return run_latent_prefill(args)
    return run_decode(args)


def secondary_runs(args):
    """Short runs of the other workloads (config3 prefill, config5 block-float-8 decode, config4
    large decode with its chunked-prefill pass, latent decode) in the headline's process, so that
    their figures come under the same clock: the same functions as `--workload ...`, fewer steps,
    only the key figures."""
    import copy
    import gc

    import torch

    out = {}
    for wl, steps, warmup in (("config3", 96, 8), ("config5", 96, 12), ("config4", 32, 4), ("latent", 96, 8),
                              ("latent128", 32, 4), ("latent-prefill", 32, 4)):
        gc.collect()
        torch.cuda.empty_cache()
        sub = copy.copy(args)
        sub.workload, sub.steps, sub.warmup = wl, steps, warmup
        if wl == "config4":
            sub.rotate = 1  # one copy of the 128-user pool is already far beyond the caches
        r = run_workload(sub)
        keep = {k: r[k] for k in ("metric", "value", "unit", "steps", "warmup", "ms_per_step", "ms_per_step_min",
                                  "ms_per_step_max", "dtype", "roofline")}
        keep["workload"] = r["config"]["workload"]
        for extra in ("pct_of_hbm_peak", "chunk_pass"):
            if extra in r:
                keep[extra] = r[extra]
        out[wl] = keep
    gc.collect()
    torch.cuda.empty_cache()
    return out


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

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    if args.workload == "config3":
        out = run_prefill(args)
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_prefill_baseline(args)
    elif args.workload.startswith("latent"):
        out = run_workload(args)  # (no CPU leg: the headline workload carries it)
    else:
        out = run_decode(args)
        if args.workload == "config2" and not args.no_secondary:
            out["secondary"] = secondary_runs(args)
        if not args.no_cpu_baseline:
            out["cpu_baseline"] = cpu_decode_baseline(args)
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").random_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        out["calibration"] = {"kernel": "torch device copy", "bytes_read": 256 << 20, "bytes_written": 256 << 20}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
