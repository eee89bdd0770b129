"""Seeded synthetic workloads of the paged-attention path (the shapes the benchmark and
the parity tests run).  Everything is generated on the CPU from one ``torch.Generator``
and moved to the requested device by the caller, so the CPU checker and the GPU kernels
see identical bits.

The generators reproduce the invariants of the reference's host metadata
(vllm_tt/model_runner.py:1727-1741, 1945-1985): ``cache_position`` is the position of the
token written this step, page-table rows list a user's blocks in logical order and are
zero beyond them, block 0 is the null block.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import torch


@dataclass
class DecodeWorkload:
    name: str
    q: torch.Tensor  # [1, B, Hq, D] bf16
    k_new: torch.Tensor  # [1, B, Hkv, D] bf16 (token written this step)
    v_new: torch.Tensor
    k_cache: torch.Tensor  # [NB, Hkv, bs, D] bf16
    v_cache: torch.Tensor
    page_table: torch.Tensor  # [B, W] int32
    cache_position: torch.Tensor  # [B] int32 = context length before this step
    scale: float

    @property
    def shape(self):
        nb, hkv, bs, d = self.k_cache.shape
        return dict(users=self.q.shape[1], q_heads=self.q.shape[2], kv_heads=hkv, head_size=d,
                    block_size=bs, num_blocks=nb, table_width=self.page_table.shape[1])

    def to(self, device):
        return DecodeWorkload(self.name, *[
            t.to(device) for t in (self.q, self.k_new, self.v_new, self.k_cache, self.v_cache,
                                   self.page_table, self.cache_position)
        ], self.scale)

    def decode_bytes(self, kv_bytes_per_elem: float = 2.0) -> int:
        """Algorithmic HBM bytes of one decode-attention launch: every attended K and V
        element once per KV head, q read, output written, page-table entries and
        positions read."""
        s = self.shape
        attended = (self.cache_position.to(torch.int64) + 1).clamp(min=0)
        kv = int(attended.sum()) * s["kv_heads"] * s["head_size"] * 2 * kv_bytes_per_elem
        qo = 2 * s["users"] * s["q_heads"] * s["head_size"] * 2
        tables = int(((attended + s["block_size"] - 1) // s["block_size"]).sum()) * 4 + s["users"] * 4
        return int(kv + qo + tables)

    def update_bytes(self) -> int:
        """One-token K and V writes: row read + row written, two tensors."""
        s = self.shape
        return 2 * 2 * s["users"] * s["kv_heads"] * s["head_size"] * 2


def _randn_bf16(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


def decode_config1(seed: int = 1) -> DecodeWorkload:
    """Batch 1, 8/8 heads, head 64, block 32, context 128: the reference's CPU-runnable
    case.  The cache is pre-filled for 128 tokens through a random permutation of the 16
    physical blocks; the new token goes to position 128."""
    g = torch.Generator().manual_seed(seed)
    b, hq, hkv, d, bs, nb, ctx = 1, 8, 8, 64, 32, 16, 128
    table = torch.randperm(nb, generator=g).view(1, nb).to(torch.int32)
    k_cache = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16)
    v_cache = torch.zeros(nb, hkv, bs, d, dtype=torch.bfloat16)
    k_ctx = _randn_bf16(g, hkv, ctx, d)
    v_ctx = _randn_bf16(g, hkv, ctx, d)
    for t in range(ctx):
        k_cache[table[0, t // bs], :, t % bs] = k_ctx[:, t]
        v_cache[table[0, t // bs], :, t % bs] = v_ctx[:, t]
    return DecodeWorkload(
        "config1-b1-h8x8-d64-bs32-ctx128",
        _randn_bf16(g, 1, b, hq, d), _randn_bf16(g, 1, b, hkv, d), _randn_bf16(g, 1, b, hkv, d),
        k_cache, v_cache, table, torch.tensor([ctx], dtype=torch.int32), 1.0 / math.sqrt(d),
    )


def decode_ragged(
    name: str,
    seed: int,
    users: int,
    q_heads: int,
    kv_heads: int,
    head_size: int,
    block_size: int,
    num_blocks: int,
    context: List[int],
    table_width: Optional[int] = None,
    cache_fill: str = "randn",
    cache_device: Optional[str] = None,
) -> DecodeWorkload:
    """Ragged decode batch: user u has ``context[u]`` tokens cached and writes position
    ``context[u]``; its blocks are a disjoint slice of a random permutation of the pool
    (block 0 is kept out as the null block), zero-padded to ``table_width``.
    ``cache_device`` draws the cache contents on that device instead of the CPU (for
    benchmarks of full-size pools, where the values only need to be N(0, 1))."""
    g = torch.Generator().manual_seed(seed)
    need = [(c + 1 + block_size - 1) // block_size for c in context]
    assert sum(need) <= num_blocks - 1, "pool too small"
    width = table_width or (max(need) + 7) // 8 * 8
    perm = torch.randperm(num_blocks - 1, generator=g) + 1
    table = torch.zeros(users, width, dtype=torch.int32)
    at = 0
    for u, n in enumerate(need):
        table[u, :n] = perm[at : at + n].to(torch.int32)
        at += n
    shape = (num_blocks, kv_heads, block_size, head_size)
    if cache_fill == "randn" and cache_device is not None:
        dg = torch.Generator(device=cache_device).manual_seed(seed)
        k_cache = torch.randn(shape, generator=dg, device=cache_device, dtype=torch.bfloat16)
        v_cache = torch.randn(shape, generator=dg, device=cache_device, dtype=torch.bfloat16)
    elif cache_fill == "randn":
        # generated in slices so peak host memory stays near one cache
        k_cache = torch.empty(shape, dtype=torch.bfloat16)
        v_cache = torch.empty(shape, dtype=torch.bfloat16)
        step = max(1, (1 << 24) // (kv_heads * block_size * head_size))
        for s in range(0, num_blocks, step):
            e = min(num_blocks, s + step)
            k_cache[s:e] = torch.randn(e - s, *shape[1:], generator=g).to(torch.bfloat16)
            v_cache[s:e] = torch.randn(e - s, *shape[1:], generator=g).to(torch.bfloat16)
    else:
        k_cache = torch.zeros(shape, dtype=torch.bfloat16)
        v_cache = torch.zeros(shape, dtype=torch.bfloat16)
    return DecodeWorkload(
        name,
        _randn_bf16(g, 1, users, q_heads, head_size),
        _randn_bf16(g, 1, users, kv_heads, head_size),
        _randn_bf16(g, 1, users, kv_heads, head_size),
        k_cache, v_cache, table, torch.tensor(context, dtype=torch.int32),
        1.0 / math.sqrt(head_size),
    )


def decode_config2(seed: int = 2, users: int = 32, num_blocks: int = 4096,
                   cache_device: Optional[str] = None) -> DecodeWorkload:
    """Llama-3-8B shape: 32/8 heads, head 128, block 64, batch 32, context uniform in
    [512, 4096], blocks drawn without reuse from a pool of 4096."""
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(512, 4097, (users,), generator=g).tolist()
    return decode_ragged("config2-llama3-8b-b32-h32x8-d128-bs64-ctx512..4096", seed + 1000, users,
                         32, 8, 128, 64, num_blocks, ctx, table_width=72,
                         cache_device=cache_device)


def fragmented_block_order(gen: torch.Generator, num_blocks: int, rounds: int = 4) -> List[int]:
    """Order in which a block pool hands out blocks after a seeded history of interleaved
    allocations and frees (free list = queue, freed blocks return to its tail, as in vLLM's
    block pool).  Block 0 stays reserved as the null block."""
    free = list(range(1, num_blocks))
    live: List[List[int]] = []
    for _ in range(rounds):
        # allocate variable-length requests until ~85% of the pool is in use
        while len(free) > 0.15 * num_blocks:
            n = int(torch.randint(1, 96, (1,), generator=gen))
            n = min(n, len(free))
            live.append(free[:n])
            del free[:n]
        # free a random half of the live requests, in random order
        order = torch.randperm(len(live), generator=gen).tolist()
        keep = []
        for j, idx in enumerate(order):
            if j % 2 == 0:
                free.extend(live[idx])
            else:
                keep.append(live[idx])
        live = keep
    order = torch.randperm(len(live), generator=gen).tolist()
    for idx in order:
        free.extend(live[idx])
    return free


def decode_config4(seed: int = 4, users: int = 128, num_blocks: int = 16384,
                   cache_device: Optional[str] = None) -> DecodeWorkload:
    """Llama-3-70B shape on one GPU: 64/8 heads, head 128, block 64, batch 128, context
    log-uniform in [256, 32768]; block tables come out of a pool fragmented by interleaved
    allocations and frees, so they are non-contiguous and interleaved between users."""
    g = torch.Generator().manual_seed(seed)
    u = torch.rand(users, generator=g)
    ctx = torch.exp(math.log(256) + u * (math.log(32768) - math.log(256))).round().long()
    ctx = ctx.clamp(256, 32767).tolist()
    wl = decode_ragged("config4-llama3-70b-b128-h64x8-d128-bs64-ctx256..32768", seed + 1000,
                       users, 64, 8, 128, 64, num_blocks, ctx, table_width=520,
                       cache_device=cache_device)
    order = fragmented_block_order(g, num_blocks)
    need = [(c + 1 + 63) // 64 for c in ctx]
    assert sum(need) <= len(order), "pool too small"
    # users grow in round-robin bursts, like requests decoding side by side
    table = torch.zeros_like(wl.page_table)
    have = [0] * users
    at = 0
    while any(h < n for h, n in zip(have, need)):
        for uu in range(users):
            burst = min(4, need[uu] - have[uu])
            for _ in range(burst):
                table[uu, have[uu]] = order[at]
                have[uu] += 1
                at += 1
    wl.page_table = table
    return wl


@dataclass
class PrefillWorkload:
    name: str
    q: torch.Tensor  # [users * S, Hq * D] token-major, as the attention layer hands it over
    k: torch.Tensor  # [users * S, Hkv * D]
    v: torch.Tensor
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    page_table: torch.Tensor  # [users, W]
    fill_page_table: torch.Tensor
    batch_idx: torch.Tensor
    chunk_start: Optional[torch.Tensor]  # [1] int32 or None (first chunk)
    users: int
    seq: int
    q_heads: int
    kv_heads: int
    head_size: int

    def to(self, device):
        mv = lambda t: None if t is None else t.to(device)  # noqa: E731
        return PrefillWorkload(self.name, mv(self.q), mv(self.k), mv(self.v), mv(self.k_cache),
                               mv(self.v_cache), mv(self.page_table), mv(self.fill_page_table),
                               mv(self.batch_idx), mv(self.chunk_start), self.users, self.seq,
                               self.q_heads, self.kv_heads, self.head_size)

    def useful_flops(self) -> float:
        """4 * D * Hq * sum over users of (Lc * start + Lc (Lc + 1) / 2): the causal part only."""
        start = 0 if self.chunk_start is None else int(self.chunk_start[0])
        lc = self.seq
        return 4.0 * self.head_size * self.q_heads * self.users * (lc * start + lc * (lc + 1) / 2)

    def fill_bytes(self) -> int:
        return 2 * 2 * self.users * self.seq * self.kv_heads * self.head_size * 2


def prefill_workload(name: str, seed: int, users: int, seq: int, q_heads: int, kv_heads: int,
                     head_size: int, block_size: int, start: int = 0,
                     device: Optional[str] = None) -> PrefillWorkload:
    """`users` prompts (or continuation chunks after `start` cached tokens, start a multiple of
    the block size) of `seq` tokens; blocks from a random permutation of the pool."""
    dev = device or "cpu"
    g = torch.Generator(device=dev).manual_seed(seed)
    cg = torch.Generator().manual_seed(seed)
    assert start % block_size == 0
    w = (start + seq + block_size - 1) // block_size
    w = (w + 7) // 8 * 8
    nb = users * w + 1
    table = (torch.randperm(nb - 1, generator=cg) + 1).view(users, w).to(torch.int32)
    mk = lambda *sh: torch.randn(*sh, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)  # noqa: E731
    shape = (nb, kv_heads, block_size, head_size)
    if start:
        k_cache, v_cache = mk(*shape), mk(*shape)
    else:
        k_cache = torch.zeros(shape, dtype=torch.bfloat16, device=dev)
        v_cache = torch.zeros(shape, dtype=torch.bfloat16, device=dev)
    return PrefillWorkload(
        name, mk(users * seq, q_heads * head_size), mk(users * seq, kv_heads * head_size),
        mk(users * seq, kv_heads * head_size), k_cache, v_cache, table,
        torch.roll(table, -(start // block_size), dims=1),
        torch.arange(users, dtype=torch.int32),
        torch.tensor([start], dtype=torch.int32) if start else None,
        users, seq, q_heads, kv_heads, head_size,
    )


def prefill_config3(seed: int = 3, device: Optional[str] = None) -> PrefillWorkload:
    """Causal prefill at the Llama-3-8B head shape: 4 prompts of 2048 tokens, 32/8 heads,
    head 128, block 64."""
    return prefill_workload("config3-llama3-8b-prefill-b4x2048-h32x8-d128-bs64", seed, 4, 2048,
                            32, 8, 128, 64, 0, device)


def prefill_config4_chunks(seed: int = 44, device: Optional[str] = None) -> PrefillWorkload:
    """The chunked-prefill pass of the 70B configuration: 4 sequences, 512-token chunks on top
    of 4096 cached tokens, 64/8 heads."""
    return prefill_workload("config4-chunks-b4x512-start4096-h64x8-d128-bs64", seed, 4, 512, 64,
                            8, 128, 64, 4096, device)


def add_outlier_channels(wl: DecodeWorkload, seed: int, fraction: float = 0.01, gain: float = 20.0):
    """Scales a random `fraction` of the (kv_head, head_dim) channels of K and V (cache and new
    token) by `gain`: the outlier-channel distribution of the block-float-8 configuration."""
    g = torch.Generator().manual_seed(seed)
    _, hkv, _, d = wl.k_cache.shape
    n = max(1, int(round(fraction * hkv * d)))
    for cache, new in ((wl.k_cache, wl.k_new), (wl.v_cache, wl.v_new)):
        ch = torch.randperm(hkv * d, generator=g)[:n]
        hh, dd = (ch // d).to(cache.device), (ch % d).to(cache.device)
        cache[:, hh, :, dd] = (cache[:, hh, :, dd].float() * gain).to(cache.dtype)
        new[:, :, hh.cpu(), dd.cpu()] = (new[:, :, hh.cpu(), dd.cpu()].float() * gain).to(new.dtype)
    return wl


def decode_config5(seed: int = 5, users: int = 32, num_blocks: int = 4096,
                   cache_device: Optional[str] = None) -> DecodeWorkload:
    """The Llama-3-8B decode shape with N(0, 1) K/V where 1% of the channels are scaled x20.
    The caches are returned in bfloat16; the caller packs them to block-float-8."""
    g = torch.Generator().manual_seed(seed)
    ctx = torch.randint(512, 4097, (users,), generator=g).tolist()
    wl = decode_ragged("config5-llama3-8b-bfp8-b32-h32x8-d128-bs64-ctx512..4096", seed + 1000,
                       users, 32, 8, 128, 64, num_blocks, ctx, table_width=72,
                       cache_device=cache_device)
    return add_outlier_channels(wl, seed + 2000)
