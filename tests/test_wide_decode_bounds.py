"""Host-side model of the address arithmetic of the latent decode kernel
(tt-xla_amd/csrc/decode_wide.hip): for every shape that tests/test_gpu_mla.py runs, every global
source range, LDS-DMA destination, LDS operand read and partial-slot write the kernel forms must
stay inside the buffer it belongs to.  LDS-DMA destinations are modelled as the instruction takes
them: ABSOLUTE byte addresses in the workgroup's LDS allocation (the static arrays come first, the
dynamic stages behind them), 16-byte aligned, never inside the static arrays and never past the
CU's LDS.  Pure integer arithmetic, no GPU: it restates the kernel's formulas, so it guards the
geometry (strides, tile sizes, slot layout), not the generated code."""

import itertools

import pytest

import test_gpu_mla as G

K_TILE = 64
STATIC_LDS = 8224          # s_pref + s_len + s_wsum of the kernel
LDS_PER_CU = 160 * 1024

SHAPES = [
    # head_size, head_dim_v, separate_v, heads, kv_heads, block_size, table_width, num_blocks, users
    (576, 512, False, 16, 1, 32, 24, 96, 4),
    (576, 512, False, 128, 1, 64, 12, 36, 3),
    (192, 128, False, 16, 1, 32, 16, 128, 8),
    (192, 128, False, 16, 4, 32, 16, 128, 8),
    (128, 128, True, 8, 8, 32, 16, 128, 8),
    (128, 64, True, 16, 1, 32, 16, 128, 8),
    (192, 128, False, 8, 1, 1184, 1, 1, 1024),   # prefill mapping: one block of s tokens
    (576, 512, False, 16, 1, 32, 8, 24, 3),      # test_mla_decode_padded_row_sink_and_errors
    (576, 512, False, 16, 1, 32, 3, 12, 2),      # test_mla_backend_prefill_then_decode, decode step
    (576, 512, False, 16, 1, 64, 1, 1, 64),      # ... its prefill (64 tokens per user)
]
# every case of the GPU test's own lists
SHAPES += [(dh, dv, has_v, hq, nkv, bs, width, width * users, users)
           for users, hq, nkv, dh, dv, has_v, bs, width, _ in G.DECODE]
# prefill with a separate V runs on the decode kernels: query row i is a user, the sequence one block
# of s tokens, at most 1024 users per launch
SHAPES += [(dh, dv, has_v, hq, nkv, s, 1, 1, min(s, 1024)) for _, hq, s, dh, nkv, dv, has_v in G.PREFILL]
SHAPES = sorted(set(SHAPES))
BUILT_16 = {(576, 512), (576, 384), (192, 128), (128, 128)}


def _form_128(shape):
    """Shapes the 128-head form takes from the workgroup-shared one: V from K, more than 16 heads per
    KV head in segments of up to 128, 16-row pieces inside one block."""
    dqk, dv, sep_v, hq, nkv, bs = shape[:6]
    g = hq // nkv
    return not sep_v and (dqk, dv) in BUILT_16 and bs % 16 == 0 and g > 16 and (g <= 128 or g % 128 == 0)


SHAPES_128 = [s for s in SHAPES if _form_128(s)]
SHAPES = [s for s in SHAPES if not _form_128(s)] + [(576, 512, False, 128, 1, 64, 12, 36, 3), (128, 128, False, 32, 1, 32, 16, 128, 8)]


def _geometry(hq, nkv):
    g = hq // nkv
    if g <= 32:
        return 1, g
    assert g % 32 == 0
    return g // 32, 32


@pytest.mark.parametrize("dqk,dv,sep_v,hq,nkv,bs,width,nb,users", SHAPES)
def test_every_address_stays_in_bounds(dqk, dv, sep_v, hq, nkv, bs, width, nb, users):
    dvw = 128 if dv % 128 == 0 else 64
    n_slices = dv // dvw
    assert dv % dvw == 0 and n_slices <= (2 if sep_v else 4)
    nhb, gseg = _geometry(hq, nkv)
    krow = 2 * dqk + 16
    ktile = K_TILE * krow
    vrow_max = 2 * 2 * dvw + 16
    vtile = K_TILE * vrow_max if sep_v else 0
    stage = ktile + vtile
    assert STATIC_LDS + 2 * stage <= LDS_PER_CU, "two stages must fit the CU's LDS"
    row_bytes = 2 * dqk
    cache_bytes = nb * nkv * bs * dqk * 2
    vcache_bytes = nb * nkv * bs * dv * 2
    v_lds_row = 2 * dv + 16
    assert v_lds_row <= vrow_max or not sep_v

    cap = width * bs
    for t in {0, (cap - 1) // K_TILE}:                      # first and last tile of a full table
        for phys, kvh in itertools.product({0, nb - 1}, {0, nkv - 1}):
            for r in (0, 15, 16, 63):                      # rows moved by different wavefronts
                tk = t * K_TILE + r
                col = tk // bs
                p = phys if col < width else 0            # columns past the table read block 0
                row = (p * nkv + kvh) * bs + (tk - col * bs)
                src = row * dqk * 2
                # the row index inside a block must be < block_size
                assert 0 <= tk - col * bs < bs
                assert 0 <= src and src + row_bytes <= cache_bytes
                assert src % 16 == 0
                for buf in (0, 1):
                    dst = STATIC_LDS + buf * stage + r * krow      # absolute, as M0 carries it
                    assert dst % 16 == 0 and dst >= STATIC_LDS
                    assert dst + row_bytes <= STATIC_LDS + buf * stage + ktile <= LDS_PER_CU
                    # the row moves as whole 1 KiB pieces (64 lanes x 16 bytes) plus a tail under a
                    # lane mask: together exactly the row, nothing beyond it
                    full, rem_lanes = row_bytes // 1024, (row_bytes % 1024) // 16
                    assert full * 1024 + rem_lanes * 16 == row_bytes and rem_lanes < 64
                    if sep_v:
                        vsrc = row * dv * 2
                        assert vsrc + 2 * dv <= vcache_bytes
                        vdst = STATIC_LDS + buf * stage + ktile + r * v_lds_row
                        assert vdst % 16 == 0 and vsrc % 16 == 0 and 2 * dv <= 1024
                        assert vdst + 2 * dv <= STATIC_LDS + (buf + 1) * stage <= LDS_PER_CU

    # LDS operand reads of every lane
    ksteps = dqk // 16
    for lane in range(64):
        n, h = lane & 31, lane >> 5
        for kb in (0, 1):
            for s in (0, ksteps - 1):
                off = (32 * kb + n) * krow + 16 * h + 32 * s
                assert off + 16 <= ktile and off + 16 <= (32 * kb + n) * krow + row_bytes
        grp, a16 = lane >> 4, lane & 15
        vstride = v_lds_row if sep_v else krow
        for wave in range(n_slices):
            base = (4 * (grp >> 1) + (a16 >> 2)) * vstride + 2 * (wave * dvw + 16 * (grp & 1) + 4 * (a16 & 3))
            for kb, s, db, hi in itertools.product((0, 1), (0, 1), range(dvw // 32), (0, 1)):
                off = base + (32 * kb + 16 * s) * vstride + 64 * db + hi * 8 * vstride
                row = off // vstride
                assert row < K_TILE
                assert off % vstride + 8 <= 2 * dv, "V fragment must stay inside the value columns"

    # partial slots and workspace
    slot_floats = (gseg * dv + 2 * gseg + 3) // 4 * 4
    for n in range(gseg):
        for wave in range(n_slices):
            for h in (0, 1):
                last = n * dv + wave * dvw + 4 * h + 32 * (dvw // 32 - 1) + 8 * 3 + 3
                assert last < gseg * dv
        assert gseg * dv + gseg + n < slot_floats
    segs = users * nkv * nhb
    cus = 256
    # slot index = workgroup + segment; workgroups that get work < cus
    assert (cus - 1) + (segs - 1) < cus + segs
    # head index of (segment, column) stays a query head
    for seg_h in (0, nkv * nhb - 1):
        assert seg_h * gseg + gseg - 1 < hq
        assert seg_h // nhb < nkv


# ---- the 16-head form (every wavefront streams its own 16-token tiles) ---------------------------
SHAPES_16 = [s for s in SHAPES
             if not s[2] and s[3] // s[4] <= 16 and s[5] % 16 == 0 and (s[0], s[1]) in BUILT_16]


def test_the_16_head_form_is_exercised():
    assert len(SHAPES_16) >= 6
    assert any(s[0] == 576 for s in SHAPES_16) and any(s[0] == 192 for s in SHAPES_16)


def _position(row_bytes, r, c):
    """LDS chunk position of chunk c of row r (the kernel's Latent16::position)."""
    half_period = (row_bytes // 4) % 64 == 32
    r &= 15
    m = (r >> 1) & 7
    if half_period:
        return c ^ ((((m & 3) << 1) | (m >> 2)) ^ ((m >> 2) << 2))
    return c ^ ((((r & 7) ^ ((r >> 3) << 2)) << 1) | (r >> 3))


# lanes the LDS serves in one cycle (measured on gfx950 with pairs of active lanes and the bank-conflict
# counter): 16-byte reads in four groups of 16, 8-byte reads in two groups of 32
B128_GROUPS = [[0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27],
               [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31]]
B128_GROUPS += [[l + 32 for l in g] for g in B128_GROUPS]
B64_GROUPS = [list(range(32)), list(range(32, 64))]


@pytest.mark.parametrize("dqk,dv", sorted(BUILT_16))
def test_fragment_reads_find_their_lanes_in_different_banks(dqk, dv):
    """64 banks of 4 bytes.  A-operand read of the score product: lane (n, quad) reads 16 bytes of row n.
    Transposing read of the value columns: lane (n, quad) reads 8 bytes of row 4 quad + n / 4."""
    row_bytes = 2 * dqk
    for s in range(dqk // 32):
        for group in B128_GROUPS:
            banks = []
            for lane in group:
                n, quad = lane & 15, lane >> 4
                off = n * row_bytes + 16 * _position(row_bytes, n, 4 * s + quad)
                banks += [(off // 4 + w) % 64 for w in range(4)]
            assert len(set(banks)) == 64, (s, group)
    for vb in range(dv // 16):
        for group in B64_GROUPS:
            banks = []
            for lane in group:
                n, quad = lane & 15, lane >> 4
                rv, q = 4 * quad + (n >> 2), n & 3
                off = rv * row_bytes + 16 * _position(row_bytes, rv, 2 * vb + (q >> 1)) + 8 * (q & 1)
                banks += [(off // 4) % 64, (off // 4 + 1) % 64]
            assert len(set(banks)) == 64, (vb, group)


@pytest.mark.parametrize("dqk,dv,sep_v,hq,nkv,bs,width,nb,users", SHAPES_16)
def test_every_address_of_the_16_head_form_stays_in_bounds(dqk, dv, sep_v, hq, nkv, bs, width, nb, users):
    tile, waves = 16, 4
    g = hq // nkv
    row_bytes = 2 * dqk
    cpr = row_bytes // 16
    stage = tile * row_bytes
    wave_lds = 2 * stage
    ndma = stage // 1024
    assert stage % 1024 == 0 and STATIC_LDS + waves * wave_lds <= LDS_PER_CU
    assert (row_bytes // 4) % 64 in (0, 32) and cpr % (8 if (row_bytes // 4) % 64 == 32 else 16) == 0
    cache_bytes = nb * nkv * bs * row_bytes
    # the swizzle permutes the chunks of a row among themselves
    for r in range(tile):
        assert sorted(_position(row_bytes, r, c) for c in range(cpr)) == list(range(cpr))
    cap = width * bs
    for t in {0, (cap - 1) // tile}:
        tok0 = t * tile
        col = tok0 // bs
        assert tok0 - col * bs + tile <= bs, "a tile lies inside one block"
        for phys, kvh in itertools.product({0, nb - 1}, {0, nkv - 1}):
            tile_base = ((phys * nkv + kvh) * bs + (tok0 - col * bs)) * row_bytes
            assert tile_base % 16 == 0
            seen = set()
            for k in range(ndma):
                for lane in range(64):
                    pos = 64 * k + lane
                    r, p = pos // cpr, pos % cpr
                    off = r * row_bytes + 16 * _position(row_bytes, r, p)
                    assert 0 <= off and off + 16 <= stage and tile_base + off + 16 <= cache_bytes
                    seen.add(off)
                for wib, buf in itertools.product(range(waves), (0, 1)):
                    dst = STATIC_LDS + wib * wave_lds + buf * stage + 1024 * k     # absolute, as M0 carries it
                    assert dst % 16 == 0 and dst + 1024 <= STATIC_LDS + wib * wave_lds + (buf + 1) * stage <= LDS_PER_CU
            assert len(seen) == stage // 16, "every chunk of the tile is fetched exactly once"
    ksteps, vb = dqk // 32, dv // 16
    assert dqk % 32 == 0 and dv % 16 == 0 and dv <= dqk
    for s in range(ksteps):
        for quad in range(4):                                      # 16 lanes of an A-operand read: 16 bank quads
            quads = {((n * row_bytes + 16 * _position(row_bytes, n, 4 * s + quad)) // 16) % 16 for n in range(16)}
            assert len(quads) == 16
    for lane in range(64):
        n, quad = lane & 15, lane >> 4
        for s in (0, ksteps - 1):
            off = n * row_bytes + 16 * _position(row_bytes, n, 4 * s + quad)
            assert off // row_bytes == n and off + 16 <= stage
        rv, q = 4 * quad + (n >> 2), n & 3
        for b in (0, vb - 1):
            off = rv * row_bytes + 16 * _position(row_bytes, rv, 2 * b + (q >> 1)) + 8 * (q & 1)
            assert off // row_bytes == rv and off + 8 <= stage
        assert 8 * quad + 32 * (ksteps - 1) + 8 <= dqk
        slot_floats = (g * dv + 2 * g + 3) // 4 * 4
        # bfloat16 partials: one block of 16 heads x 16 columns per block of columns
        slot_floats_bf16 = (16 * dv // 2 + 2 * g + 3) // 4 * 4
        if n < g:
            assert n * dv + 4 * quad + 16 * (vb - 1) + 4 <= g * dv
            assert g * dv + g + n < slot_floats
            assert (128 * (vb - 1) + 8 * n + 2 * quad) + 2 <= 16 * dv // 2 and 16 * dv // 2 + g + n < slot_floats_bf16
    segs, cus = users * nkv, 256
    assert (waves * cus - 1) + (segs - 1) < waves * cus + segs     # slot index = wavefront + segment


# ---- the 128-head form and the prefill kernel: four wavefronts on shared steps of two 16-row pieces ----
STEP_KEYS, STAGES, WAVES_SHARED, WAVE_ROWS = 32, 4, 4, 32


def _shared_step_checks(dqk, dv):
    """What both kernels share: a ring of four stages, each the two pieces of a step laid out like the
    16-head form's stage, every chunk of a step requested exactly once by the wavefronts' shares
    (wavefronts 2 i and 2 i + 1 fetch piece i), destinations inside the stage."""
    row_bytes, sub, npieces, waves = 2 * dqk, 16, STEP_KEYS // 16, WAVES_SHARED
    cpr = row_bytes // 16
    piece = sub * row_bytes
    ndma = piece // 1024
    stage = npieces * piece
    assert piece % 1024 == 0 and (npieces * ndma) % waves == 0
    per_wave = npieces * ndma // waves
    assert 2 * per_wave == ndma and per_wave < 16       # (the wait for a step counts the next step's requests: 4 bits)
    assert STATIC_LDS + STAGES * stage <= LDS_PER_CU
    seen = set()
    for wave in range(waves):
        for j in range(per_wave):
            k = wave * per_wave + j
            piece_i, kk = k // ndma, k % ndma
            assert piece_i == wave >> 1 and kk == (wave & 1) * per_wave + j
            for lane in range(64):
                pos = 64 * kk + lane
                rr, p = pos // cpr, pos % cpr
                assert rr < sub
                off = (sub * piece_i + rr, _position(row_bytes, rr, p))      # (row of the step, chunk of the row)
                assert off[1] < cpr
                seen.add(off)
            for i in range(STAGES):
                dst = STATIC_LDS + i * stage + 1024 * k
                assert dst % 16 == 0 and dst + 1024 <= STATIC_LDS + (i + 1) * stage <= LDS_PER_CU
    assert len(seen) == npieces * sub * cpr, "every chunk of the step is fetched exactly once"
    # fragment reads of a lane: immediate offsets of the assembly blocks stay below 64 KiB
    gc = 8 if (row_bytes // 4) % 64 == 32 else 16
    assert piece + 16 * gc * (dqk // 32 // (gc // 4)) < 65536 and piece + 16 * gc * (dv // 16 // (gc // 2)) < 65536
    return row_bytes, piece, stage, per_wave, ndma


def test_the_128_head_form_is_exercised():
    assert any(s[3] // s[4] == 128 for s in SHAPES_128) and any(s[3] // s[4] % 16 for s in SHAPES_128)
    assert any(s[3] // s[4] > 128 for s in SHAPES_128)


@pytest.mark.parametrize("dqk,dv,sep_v,hq,nkv,bs,width,nb,users", SHAPES_128)
def test_every_address_of_the_128_head_form_stays_in_bounds(dqk, dv, sep_v, hq, nkv, bs, width, nb, users):
    row_bytes, piece, stage, per_wave, ndma = _shared_step_checks(dqk, dv)
    g = hq // nkv
    nhb, gseg = (1, g) if g <= 128 else (g // 128, 128)
    assert nhb * gseg == g
    cache_bytes = nb * nkv * bs * row_bytes
    cap = width * bs
    for t, half in itertools.product({0, (cap - 1) // K_TILE}, (0, 1)):
        for wave in range(WAVES_SHARED):
            tok0 = t * K_TILE + STEP_KEYS * half + 16 * (wave >> 1)
            col = tok0 // bs
            assert tok0 - col * bs + 16 <= bs, "a piece lies inside one block"
            for phys, kvh in itertools.product({0, nb - 1}, {0, nkv - 1}):
                p = phys if col < width else 0
                base = ((p * nkv + kvh) * bs + (tok0 - col * bs)) * row_bytes
                assert base % 16 == 0 and base + piece <= cache_bytes
    vb = dv // 16
    slot_floats = (gseg * dv + 2 * gseg + 3) // 4 * 4
    # bfloat16 partials lie in blocks of 16 heads x 16 columns, the last block of heads padded
    vals_bf16 = (gseg + 15) // 16 * 16 * dv // 2
    slot_floats_bf16 = (vals_bf16 + 2 * gseg + 3) // 4 * 4
    assert slot_floats_bf16 <= slot_floats, "the workspace is sized for float partials"
    words = set()
    for wave, rb, n, quad in itertools.product(range(WAVES_SHARED), (0, 1), range(16), range(4)):
        hg = WAVE_ROWS * wave + 16 * rb + n
        if hg < gseg:
            assert hg * dv + 4 * quad + 16 * (vb - 1) + 4 <= gseg * dv
            assert gseg * dv + gseg + hg < slot_floats
            assert vals_bf16 + gseg + hg < slot_floats_bf16
            for blk in range(vb):
                w0 = (((2 * wave + rb) * vb + blk) * 16 + n) * 8 + 2 * quad
                assert w0 + 2 <= vals_bf16
                for w in (w0, w0 + 1):
                    assert w not in words
                    words.add(w)
                    # what the merge kernel makes of the word: the head and the first of its two columns
                    b, inb = w >> 7, w & 127
                    assert (16 * (b // vb) + (inb >> 3), 16 * (b % vb) + 2 * (inb & 7)) == (hg, 16 * blk + 4 * quad + 2 * (w - w0))
    assert len(words) == gseg * dv // 2
    # the merge's threads of four words: aligned, inside one head's eight, 16-byte output pieces
    assert slot_floats_bf16 % 4 == 0 and vals_bf16 % 4 == 0
    for w0 in range(0, vals_bf16, 4):
        heads = {16 * ((w >> 7) // vb) + ((w & 127) >> 3) for w in range(w0, w0 + 4)}
        cols = [16 * ((w >> 7) % vb) + 2 * (w & 7) for w in range(w0, w0 + 4)]
        assert len(heads) == 1 and cols[0] % 8 == 0 and cols == list(range(cols[0], cols[0] + 8, 2))
    for seg_h in (0, nkv * nhb - 1):
        assert seg_h * gseg + gseg - 1 < hq and seg_h // nhb < nkv
    segs, cus = users * nkv * nhb, 256
    assert segs <= (cus + 1) * 256, "one thread of the grid publishes each segment's partial slots"


PREFILL_SHAPES = [(dh, dv, hq, nkv, s, b) for b, hq, s, dh, nkv, dv, has_v in G.PREFILL + G.MASKED_PREFILL
                  if not has_v and (dh, dv) in {(576, 512), (192, 128), (128, 128)}]


@pytest.mark.parametrize("dqk,dv,hq,nkv,s,batch", sorted(set(PREFILL_SHAPES)))
def test_every_address_of_the_prefill_kernel_stays_in_bounds(dqk, dv, hq, nkv, s, batch):
    row_bytes, piece, stage, per_wave, ndma = _shared_step_checks(dqk, dv)
    g = hq // nkv
    rows_total = g * s
    nblk = (rows_total + 127) // 128
    k_bytes = s * row_bytes                      # one (batch entry, KV head) of a contiguous K
    for blk in {0, nblk - 1}:
        last_row = min(blk * 128 + 127, rows_total - 1)
        nsteps = (last_row // g) // STEP_KEYS + 1
        for step in {0, nsteps - 1}:
            for r in (0, STEP_KEYS - 1):
                key = min(step * STEP_KEYS + r, s - 1)
                assert key * row_bytes + row_bytes <= k_bytes
        for wave, rb, n in itertools.product(range(WAVES_SHARED), (0, 1), range(16)):
            r = min(blk * 128 + WAVE_ROWS * wave + 16 * rb + n, rows_total - 1)
            t, head = r // g, r % g
            assert 0 <= t < s and head < g
            assert 32 * (dqk // 32 - 1) + 8 * 3 + 8 <= dqk and 16 * (dv // 16 - 1) + 4 * 3 + 4 <= dv
    assert batch * nkv * nblk < 2 ** 31
