"""Host-side model of the split-K schedule of the decode kernels (tt-xla_amd/csrc/decode_common.h:
build_prefix, locate_unit, publish_segment_row; the range walk that every decode kernel repeats).

The flat list holds, per (user, kv head) segment with at least one tile, `extra` leading units that
carry no work and then the segment's tiles; it is cut into n_eff equal ranges of units.  The model
restates the integer arithmetic and checks what the kernels rely on: every tile is processed by
exactly one wavefront, a wavefront's walk never leaves its range or the list, every range holds a
tile, and the (first slot, count) row published for a segment names exactly the wavefronts that
processed one of its tiles.  Pure integers, no GPU: it guards the formulas, not the generated code."""

import random

import pytest


def prefix(tiles_per_user, extra):
    pref = [0]
    for nt in tiles_per_user:
        pref.append(pref[-1] + (nt + extra if nt > 0 else 0))
    return pref


def locate(pref, hkv, x, extra):
    """-> (user, head, tile index inside the segment, tiles left, unit of that tile)"""
    lo, hi = 0, len(pref) - 2
    while lo < hi:
        mid = (lo + hi + 1) >> 1
        if pref[mid] * hkv <= x:
            lo = mid
        else:
            hi = mid - 1
    nv = pref[lo + 1] - pref[lo]
    assert nv > 0, "a unit of the list belongs to a user that has tiles"
    nt = nv - extra
    rem = x - pref[lo] * hkv
    h = rem // nv
    assert 0 <= h < hkv
    rel = max(rem - h * nv - extra, 0)
    assert 0 <= rel < nt
    return lo, h, rel, nt - rel, pref[lo] * hkv + h * nv + extra + rel


def walk(pref, hkv, n_waves, extra):
    """Tiles (user, head, rel) each wavefront processes, in order; n_eff; total."""
    total = pref[-1] * hkv
    n_eff = min(total // (extra + 1), n_waves)
    done = []
    for wave in range(n_waves):
        mine = []
        done.append(mine)
        if total == 0 or wave >= n_eff:
            continue
        x_lo, x_hi = wave * total // n_eff, (wave + 1) * total // n_eff
        u, h, rel, left, x = locate(pref, hkv, x_lo, extra)
        assert x_lo <= x < x_hi, "every range holds a tile"
        while True:
            mine.append((u, h, rel))
            nxt = x + (1 if left > 1 else 1 + extra)
            if nxt >= x_hi:
                break
            if left > 1:
                rel, left = rel + 1, left - 1
            else:
                assert x + 1 < total
                u, h, rel, left, at = locate(pref, hkv, x + 1, extra)
                assert rel == 0 and at == nxt
            x = nxt
    return done, n_eff, total


def published(pref, hkv, users, n_eff, total, extra):
    rows = {}
    for seg in range(users * hkv):
        su, sh = divmod(seg, hkv)
        snv = pref[su + 1] - pref[su]
        first = count = 0
        if snv > 0:
            x0 = pref[su] * hkv + sh * snv + extra
            x1 = x0 + (snv - extra) - 1
            w0 = ((x0 + 1) * n_eff + total - 1) // total - 1
            w1 = ((x1 + 1) * n_eff + total - 1) // total - 1
            first, count = w0 + seg, w1 - w0 + 1
        rows[seg] = (first, count)
    return rows


def check(tiles_per_user, hkv, n_waves, extra):
    users = len(tiles_per_user)
    pref = prefix(tiles_per_user, extra)
    done, n_eff, total = walk(pref, hkv, n_waves, extra)
    seen = {}
    for wave, mine in enumerate(done):
        for t in mine:
            assert t not in seen, f"tile {t} processed twice"
            seen[t] = wave
    want = {(u, h, r) for u, nt in enumerate(tiles_per_user) for h in range(hkv) for r in range(nt)}
    assert set(seen) == want
    rows = published(pref, hkv, users, n_eff, total, extra)
    for seg, (first, count) in rows.items():
        u, h = divmod(seg, hkv)
        waves = sorted({w for (tu, th, _), w in seen.items() if (tu, th) == (u, h)})
        if not waves:
            assert count == 0
            continue
        # slot of (wave, segment) is wave + segment index: a contiguous run of slots, all written
        assert waves == list(range(first - seg, first - seg + count)), (seg, waves, first, count)
        assert first + count <= n_waves + users * hkv


@pytest.mark.parametrize("extra", [0, 1, 2, 3])
def test_schedule_covers_every_tile_once(extra):
    rng = random.Random(17 + extra)
    for _ in range(60):
        users = rng.choice([1, 2, 3, 8, 32, 61])
        hkv = rng.choice([1, 2, 8])
        top = rng.choice([1, 2, 5, 40, 300])
        tiles = [rng.choice([0, rng.randint(1, top)]) if rng.random() < 0.3 else rng.randint(1, top)
                 for _ in range(users)]
        n_waves = rng.choice([4, 8, 64, 768, 1024])
        check(tiles, hkv, n_waves, extra)


@pytest.mark.parametrize("extra", [0, 1, 2])
def test_schedule_edge_cases(extra):
    check([0, 0, 0], 2, 8, extra)              # nothing attended anywhere
    check([1], 1, 1024, extra)                 # one tile, many wavefronts
    check([0, 1, 0, 0, 1, 0], 8, 768, extra)   # padded users between live ones
    check([128] * 32, 8, 768, extra)           # the Llama-3-8B shape at full context
    check([3, 1, 1, 1, 200], 1, 4, extra)      # ranges that span several short segments


def test_weighted_ranges_balance_cost():
    """With one leading unit per segment, tiles + segments opened inside a range differ by at most
    two units between wavefronts (floor of the cut, and the partly charged first segment)."""
    rng = random.Random(5)
    tiles = [rng.randint(16, 128) for _ in range(32)]
    pref = prefix(tiles, 1)
    done, n_eff, _ = walk(pref, 8, 768, 1)
    cost = []
    for mine in done[:n_eff]:
        opened = sum(1 for (_, _, rel) in mine[1:] if rel == 0)
        cost.append(len(mine) + opened)
    assert max(cost) - min(cost) <= 2
