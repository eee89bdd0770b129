#!/usr/bin/env python3
"""Writes the hand-scheduled tile loop of the prefill kernel (head size 128, four query heads of
one KV head per workgroup, 32 query rows per wavefront, two workgroups per CU) as one block of
gfx950 assembly per K / V source: build/prefill_stream_asm.h, included by prefill.hip.

Why assembly: the loop wants the matrix pipe and the vector ALU of a SIMD busy at the same time
from one instruction stream, with every register chosen by hand (256 per wavefront at two
wavefronts per SIMD) and every wait counted.  The unit of work is a BLOCK of 32 keys:

  S(i)   8 matrix instructions   S^T = K . Q^T of block i          (K fragments from LDS)
  sm(i)  ~56 vector instructions  p = exp2(s c - m), packed to bfloat16, row sum
  PV(i)  8 matrix instructions   O^T += V^T . P^T of block i       (V^T fragments from LDS)

Iteration i issues S(i + 1) and PV(i - 1) alternately, one slice of sm(i) and the LDS read of a
fragment 8 matrix instructions ahead behind each.  Scores and probabilities alternate between two
register banks by the parity of i, so nothing is copied.

The running maximum is not tracked per block.  Probabilities are taken relative to a reference
m (kept as mc = m c + 7 in the exponent domain) that only moves when some probability of the
block reaches 2, which is one OR over the packed probabilities and one test of bit 14 of every
bfloat16: p >= 2 exactly when the score exceeds the reference's maximum by 2^8, the lazy rule of
the plain loop.  The block then takes the slow path at the end of the iteration: true row maximum,
new reference, accumulators and row sum rescaled, probabilities of the block recomputed.  The first
block of a row always does (the reference starts at -inf).

Masks: a lane holds the keys key0 + 4 h + {0..3, 8..11, 16..19, 24..27} of a block (h = lane / 32)
for query row lane % 32, and may see keys up to its limit (causal diagonal, end of K / V).  Blocks
from key `mask_from` on are masked in place, at the start of their iteration, before anything reads
the scores: 16 compares of the key constants against limit - 4 h - key0 and 16 selects of -inf.
Blocks in front of it skip that with one scalar branch.

Tiles: K(t) and V(t) live in stage t & 1 of LDS (a stage = K tile, then V tile, 16 KiB each).
The barrier of tile t sits at the start of iteration 2 t + 1: K(t + 1) and V(t), requested one
barrier earlier, have landed for everyone; K(t) and V(t - 1) are not read any more, and K(t + 2),
V(t + 1) are requested into their places (LDS-DMA loads, four per tensor, wavefront and tile),
as long as such tiles exist.  Dense K / V: a tile is `stride` bytes behind the one before.  Paged
(block size a multiple of 64): a tile lies in one block; the block-table entry of tile t + 3 is
requested (a vector load, like the tiles, so one counter covers both) behind the tile requests
of barrier t and read behind barrier t + 1, where K(t + 2) needs it; V(t + 2) uses the same
offset one barrier later.  Entries outside [0, num_blocks) read block 0.

The block is entered with K(0), V(0), K(1) requested and K(0) visible (paged: and the entry of
tile 2 requested), and handles tiles 0 .. n - 1.  It leaves with the state the plain loop expects
at the top of its iteration for tile n: accumulators, row sums and reference through tile n - 1;
K(n) visible; K(n + 1) and V(n) requested where they exist.

Matrix-to-vector hazards the hardware does not interlock are kept by construction: the vector
instructions that read a score bank start two matrix instructions after the last one that wrote
it (the mask waits explicitly); a bank of probabilities is rewritten three matrix instructions
after the last one that read it; the slow path and the exit wait out the matrix pipe with s_nop.
"""

import os
import sys

PROBE = {k: bool(int(os.environ.get('PROBE_' + k, '0'))) for k in ('NOVALU', 'NOBAR', 'NODS', 'NOMFMA', 'STAMPS')}

# ---- register map (vector registers) ---------------------------------------------------------
ACC = [0, 16, 32, 48]          # output accumulators, head-dim blocks 0..3 (inputs / outputs)
QF = 64                        # Q fragments, k-step ks at QF + 4 ks (inputs)
S = [96, 112]                  # score banks
P = [128, 136]                 # probability banks (8 packed pairs each)
RING = 144                     # 8 fragment slots of 4 registers
NSLOT = 8
KOFF = 176                     # LDS byte address of the lane's K fragment, k-step ks (inputs)
VOFF = 184                     # ... of the lane's V^T fragment, output block db (inputs)
LDK = 188                      # per-lane global byte offsets of the 4 K loads of a tile (inputs)
LDV = 192                      # ... of the 4 V loads
MC, LRUN, LSUM, ALPHA = 196, 197, 198, 199   # MC, LRUN: inputs / outputs
T = [200, 201, 202, 203]
ORV, MLOC, MB, MCN = 204, 205, 206, 207
PTREQ = 208                    # paged: the requested block-table entry (input)
LIMIT = 212                    # last visible key of the lane's row, minus 4 h (input)
LIMREL, NEGINF, VZERO = 213, 214, 215
CLOBBERED = list(range(S[0], RING + 4 * NSLOT)) + list(range(LSUM, MCN + 1)) + [209, 210, 211, LIMREL, NEGINF, VZERO]

# ---- scalar registers ---------------------------------------------------------------------------
S_KBASE = "s[64:65]"           # dense: next K tile to request; paged: the K cache (both minus 3072, see dma)
S_VBASE = "s[66:67]"
S_STRIDE = "s68"               # dense: bytes from one tile to the next; paged: bytes of one (block, head) slab
S_C = "s69"                    # softmax scale times log2(e)
S_NT = "s70"                   # tiles left
S_KLEFT = "s71"                # K tiles left to request
S_M0B = "s72"                  # LDS address of this wavefront's first 1 KiB segment in stage 0's K tile
S_VLEFT = "s73"                # V tiles left to request
S_MASKFROM = "s74"             # blocks whose first key is >= this are masked
S_KEY0 = "s75"                 # first key of the block whose softmax comes next
# paged only
S_HKV, S_HK, S_NB, S_TPB = "s76", "s77", "s78", "s79"   # kv heads, this kv head, blocks in the cache, tiles per block
S_CIN = "s80"                  # tile-in-block index of the next K tile to request
S_RIN = "s81"                  # ... of the next tile whose entry is requested
S_RPTR = "s[82:83]"            # address of that entry
S_VOFF = "s[84:85]"            # byte offset in the cache of the next V tile to request
S_RLEFT = "s86"                # entries left to request
# temporaries s[87:95]
SCALAR_CLOBBERS = [f"s{r}" for r in range(87, 96)]

STAGE = 32768
VTILE = 16384
KEY_CONST = [8 * (r // 4) + r % 4 for r in range(16)]


class Out:
    def __init__(self):
        self.lines = []

    def e(self, s):
        if PROBE['NODS'] and (s.startswith('ds_read') or s.startswith('s_waitcnt lgkmcnt')):
            return
        if PROBE['NOMFMA'] and s.startswith('v_mfma'):
            return
        if PROBE['NOVALU'] and s.startswith('v_') and not s.startswith('v_mfma'):
            return
        if PROBE['NOVALU'] and s.startswith('s_cbranch_vccnz'):
            return
        if PROBE['NOBAR'] and (s.startswith('s_barrier') or s.startswith('s_waitcnt vmcnt') or s.startswith('global_load')):
            return
        self.lines.append(s)

    def label(self, name):
        self.lines.append(name + "%=:")


def vr(a, n=1):
    return f"v{a}" if n == 1 else f"v[{a}:{a + n - 1}]"


def frag_reads(frag, slot):
    """LDS read instructions of a fragment into ring slot `slot`."""
    base = RING + 4 * slot
    kind = frag[0]
    if kind == "K":
        _, stage, kb, ks = frag
        return [f"ds_read_b128 {vr(base, 4)}, v{KOFF + ks} offset:{stage * STAGE + kb * 8192}"]
    _, stage, k4, db = frag
    off = stage * STAGE + VTILE + k4 * 4096
    return [f"ds_read_b64_tr_b16 {vr(base, 2)}, v{VOFF + db} offset:{off}",
            f"ds_read_b64_tr_b16 {vr(base + 2, 2)}, v{VOFF + db} offset:{off + 2048}"]


def mfma(m, slot):
    a = vr(RING + 4 * slot, 4)
    if m[0] == "S":
        _, bank, ks = m
        d = vr(S[bank], 16)
        return f"v_mfma_f32_32x32x16_bf16 {d}, {a}, {vr(QF + 4 * ks, 4)}, {'0' if ks == 0 else d}"
    _, db, bank, k4p = m
    d = vr(ACC[db], 16)
    return f"v_mfma_f32_32x32x16_bf16 {d}, {a}, {vr(P[bank] + 4 * k4p, 4)}, {d}"


def softmax_ops(q, test=True):
    """Vector instructions of sm(i) on bank q, in an order that keeps one instruction between a
    transcendental and its first use."""
    s, p = S[q], P[q]
    A = lambda r: f"v_fma_f32 v{T[r % 4]}, v{s + r}, {S_C}, -v{MC}"
    B = lambda r: f"v_exp_f32 v{T[r % 4]}, v{T[r % 4]}"
    C = lambda j: f"v_cvt_pk_bf16_f32 v{p + j}, v{T[(2 * j) % 4]}, v{T[(2 * j + 1) % 4]}"
    D = lambda j: f"v_dot2c_f32_bf16 v{LSUM}, 0x3f803f80, v{p + j}"
    ops = [f"v_mov_b32 v{LSUM}, 0", A(0), A(1), B(0), B(1)]
    for j in range(8):
        if j < 7:
            ops += [A(2 * j + 2), A(2 * j + 3)]
        ops.append(C(j))
        if j < 7:
            ops += [B(2 * j + 2), B(2 * j + 3)]
        ops.append(D(j))
    if test:
        ops += [f"v_or3_b32 v{ORV}, v{p}, v{p + 1}, v{p + 2}",
                f"v_or3_b32 v{ORV}, v{ORV}, v{p + 3}, v{p + 4}",
                f"v_or3_b32 v{ORV}, v{ORV}, v{p + 5}, v{p + 6}",
                f"v_or_b32 v{ORV}, v{ORV}, v{p + 7}",
                f"v_and_b32 v{ORV}, 0x40004000, v{ORV}",
                f"v_cmp_ne_u32 vcc, 0, v{ORV}"]
    for i, op in enumerate(ops[:-1]):  # a transcendental's result is not read by the next instruction
        if op.startswith("v_exp_f32"):
            dst = op.split()[1].rstrip(",")
            assert dst not in [t.rstrip(",") for t in ops[i + 1].split()[2:]], (op, ops[i + 1])
    return ops


def spread(ops, nslots, first=0):
    """ops cut into nslots consecutive chunks of nearly equal size; slots before `first` get none."""
    n = nslots - first
    out = [[] for _ in range(nslots)]
    for k, op in enumerate(ops):
        out[first + (k * n) // len(ops)].append(op)
    return out


def stream(o, pairs, valu_chunks, mid=None):
    """pairs: [(matrix instruction, fragment)].  Emits the initial fragment reads (NSLOT ahead),
    then per pair: wait for its fragment, the matrix instruction, the read of the fragment NSLOT
    pairs on, the vector chunk.  `mid`: {index: callable} emitted in front of pair `index`."""
    n = len(pairs)
    issued = []  # (fragment index, instructions) in program order
    for f in range(min(NSLOT, n)):
        r = frag_reads(pairs[f][1], f % NSLOT)
        for x in r:
            o.e(x)
        issued.append((f, len(r)))
    for j in range(n):
        if mid and j in mid:
            mid[j]()
        after = sum(c for f, c in issued if f > j)
        assert after <= 15
        o.e(f"s_waitcnt lgkmcnt({after})")
        o.e(mfma(pairs[j][0], j % NSLOT))
        if j + NSLOT < n:
            r = frag_reads(pairs[j + NSLOT][1], j % NSLOT)
            for x in r:
                o.e(x)
            issued.append((j + NSLOT, len(r)))
        for x in valu_chunks[j]:
            o.e(x)


def iteration_pairs(q, kstage, kb, vstage, vk4, has_pv=True):
    """Iteration of parity q: S(i + 1) into bank 1 - q from K (kstage, key block kb), PV(i - 1)
    from bank 1 - q of the probabilities and V (vstage, key steps vk4, vk4 + 1)."""
    pairs = []
    for x in range(8):
        pairs.append((("S", 1 - q, x), ("K", kstage, kb, x)))
        if has_pv:
            pairs.append((("PV", x % 4, 1 - q, x // 4), ("V", vstage, vk4 + x // 4, x % 4)))
    return pairs


def mask_block(o, q, tag):
    """Start of the iteration whose softmax reads bank q: masks the block in place if it needs it."""
    s = S[q]
    o.e(f"s_cmp_lt_i32 {S_KEY0}, {S_MASKFROM}")
    o.e(f"s_cbranch_scc1 L_nomask_{tag}%=")
    o.e("s_nop 15")  # the last matrix instruction into this bank has written
    o.e(f"v_subrev_u32 v{LIMREL}, {S_KEY0}, v{LIMIT}")  # limit - 4 h - key0
    o.e(f"v_mov_b32 v{NEGINF}, 0xff800000")
    sel = lambda r: f"v_cndmask_b32_e64 v{s + r}, v{s + r}, v{NEGINF}, s[{88 + 2 * (r % 4)}:{89 + 2 * (r % 4)}]"
    for r in range(16):
        o.e(f"v_cmp_gt_i32_e64 s[{88 + 2 * (r % 4)}:{89 + 2 * (r % 4)}], {KEY_CONST[r]}, v{LIMREL}")
        if r >= 3:  # a select reads its mask three instructions after the compare that wrote it
            o.e(sel(r - 3))
    o.e("s_nop 1")
    for r in range(13, 16):
        o.e(sel(r))
    o.label(f"L_nomask_{tag}")
    o.e(f"s_add_u32 {S_KEY0}, {S_KEY0}, 32")


def slow_path(o, q, name, join):
    """Bank q: true row maximum, new reference, rescale, probabilities again."""
    s = S[q]
    o.label(name)
    o.e("s_nop 15")
    o.e("s_nop 15")
    o.e(f"v_max3_f32 v{MLOC}, v{s}, v{s + 1}, v{s + 2}")
    for r in range(3, 15, 2):
        o.e(f"v_max3_f32 v{MLOC}, v{MLOC}, v{s + r}, v{s + r + 1}")
    o.e(f"v_max_f32 v{MLOC}, v{MLOC}, v{s + 15}")
    o.e(f"v_mov_b32 v{MB}, v{MLOC}")
    o.e("s_nop 1")
    o.e(f"v_permlane32_swap_b32 v{MLOC}, v{MB}")
    o.e("s_nop 1")
    o.e(f"v_max_f32 v{MLOC}, v{MLOC}, v{MB}")                 # row maximum (raw score)
    o.e(f"v_fma_f32 v{MB}, v{MLOC}, {S_C}, -v{MC}")           # how far above the reference's zero
    o.e(f"v_cmp_le_f32 vcc, 1.0, v{MB}")                      # p >= 2 somewhere in the row: move
    o.e(f"v_mul_f32 v{MCN}, {S_C}, v{MLOC}")
    o.e(f"v_add_f32 v{MCN}, 0x40e00000, v{MCN}")              # m c + 7
    o.e("s_nop 1")
    o.e(f"v_cndmask_b32 v{MCN}, v{MC}, v{MCN}, vcc")
    o.e(f"v_sub_f32 v{ALPHA}, v{MC}, v{MCN}")                 # 0 where the reference stays
    o.e(f"v_exp_f32 v{ALPHA}, v{ALPHA}")
    o.e(f"v_mov_b32 v{MC}, v{MCN}")
    o.e("s_nop 0")
    o.e(f"v_mul_f32 v{LRUN}, v{LRUN}, v{ALPHA}")
    for r in range(64):
        o.e(f"v_mul_f32 v{r}, v{ALPHA}, v{r}")
    for x in softmax_ops(q, test=False):
        o.e(x)
    o.e("s_nop 4")
    o.e(f"s_branch {join}%=")


def stamp(o):
    """probe builds: wall clock (100 MHz) to the workgroup's stamp list; only where no LDS read is in flight"""
    if not PROBE['STAMPS']:
        return
    o.e("s_memrealtime s[92:93]")
    o.e("s_waitcnt lgkmcnt(0)")
    o.e("v_mov_b32 v210, s92")
    o.e("v_mov_b32 v211, s93")
    o.e("v_mov_b32 v209, s87")
    o.e("s_nop 1")
    o.e("global_store_dwordx2 v209, v[210:211], s[96:97]")
    o.e("s_add_u32 s87, s87, 8")


def four_loads(o, lane_regs, base):
    for j in range(4):
        o.e(f"global_load_lds_dwordx4 v{lane_regs + j}, {base} offset:{1024 * j}")


def dma_block(o, tp, tag, paged):
    """Requests K(t + 2) into K stage tp and V(t + 1) into V stage 1 - tp where those tiles exist.
    The instruction offset moves the LDS address as well as the global one: load j lands 1024 j
    bytes behind M0 and reads base + lane offset + 1024 j, so the lane offsets carry
    3072 - 1024 j and the bases - 3072."""
    o.e(f"s_cmp_eq_u32 {S_KLEFT}, 0")
    o.e(f"s_cbranch_scc1 L_nok_{tag}%=")
    if paged:
        o.e(f"v_readfirstlane_b32 s88, v{PTREQ}")
        o.e(f"s_cmp_lt_u32 s88, {S_NB}")
        o.e("s_cselect_b32 s88, s88, 0")
        o.e(f"s_mul_i32 s88, s88, {S_HKV}")
        o.e(f"s_add_u32 s90, s88, {S_HK}")            # block * kv_heads + kv_head
        o.e(f"s_mul_hi_u32 s89, s90, {S_STRIDE}")
        o.e(f"s_mul_i32 s88, s90, {S_STRIDE}")
        o.e(f"s_lshl_b32 s90, {S_CIN}, 14")           # 64 tokens of 256 bytes per tile inside the block
        o.e("s_add_u32 s88, s88, s90")
        o.e("s_addc_u32 s89, s89, 0")                 # s[88:89]: byte offset of tile t + 2 in a cache
        o.e("s_add_u32 s90, s64, s88")
        o.e("s_addc_u32 s91, s65, s89")
        o.e(f"s_add_u32 {S_CIN}, {S_CIN}, 1")
        o.e(f"s_cmp_eq_u32 {S_CIN}, {S_TPB}")
        o.e(f"s_cselect_b32 {S_CIN}, 0, {S_CIN}")
    o.e(f"s_add_u32 m0, {S_M0B}, {tp * STAGE}")
    o.e("s_nop 0")
    four_loads(o, LDK, "s[90:91]" if paged else S_KBASE)
    if not paged:
        o.e(f"s_add_u32 s64, s64, {S_STRIDE}")
        o.e("s_addc_u32 s65, s65, 0")
    o.e(f"s_sub_u32 {S_KLEFT}, {S_KLEFT}, 1")
    o.label(f"L_nok_{tag}")
    o.e(f"s_cmp_eq_u32 {S_VLEFT}, 0")
    o.e(f"s_cbranch_scc1 L_nov_{tag}%=")
    if paged:
        o.e("s_add_u32 s90, s66, s84")
        o.e("s_addc_u32 s91, s67, s85")
    o.e(f"s_add_u32 m0, {S_M0B}, {(1 - tp) * STAGE + VTILE}")
    o.e("s_nop 0")
    four_loads(o, LDV, "s[90:91]" if paged else S_VBASE)
    if not paged:
        o.e(f"s_add_u32 s66, s66, {S_STRIDE}")
        o.e("s_addc_u32 s67, s67, 0")
    o.e(f"s_sub_u32 {S_VLEFT}, {S_VLEFT}, 1")
    o.label(f"L_nov_{tag}")
    if paged:
        # the offset of tile t + 2 serves V one barrier later (stale only when no such V is requested)
        o.e("s_mov_b64 s[84:85], s[88:89]")
        o.e(f"s_cmp_eq_u32 {S_RLEFT}, 0")
        o.e(f"s_cbranch_scc1 L_noreq_{tag}%=")
        o.e(f"global_load_dword v{PTREQ}, v{VZERO}, {S_RPTR}")
        o.e(f"s_sub_u32 {S_RLEFT}, {S_RLEFT}, 1")
        o.e(f"s_add_u32 {S_RIN}, {S_RIN}, 1")
        o.e(f"s_cmp_lg_u32 {S_RIN}, {S_TPB}")
        o.e(f"s_cbranch_scc1 L_noreq_{tag}%=")
        o.e(f"s_mov_b32 {S_RIN}, 0")
        o.e("s_add_u32 s82, s82, 4")
        o.e("s_addc_u32 s83, s83, 0")
        o.label(f"L_noreq_{tag}")


def generate(paged):
    o = Out()
    if PROBE['STAMPS']:
        o.e("s_mov_b32 s87, 0")
    stamp(o)
    o.e(f"v_mov_b32 v{VZERO}, 0")
    # ---- S(0), then iteration 0 (no PV yet): tile 0 is in stage 0 -----------------------------
    pairs = [(("S", 0, x), ("K", 0, 0, x)) for x in range(8)] + iteration_pairs(0, 0, 1, 0, 0, has_pv=False)
    chunks = spread(softmax_ops(0), 16, first=10)
    # the mask of block 0 sits behind the second matrix instruction after S(0); it waits itself
    nop_then_mask = lambda: (o.e("s_nop 15"), mask_block(o, 0, "i0"))
    stream(o, pairs, chunks, mid={10: nop_then_mask})
    o.e("s_cbranch_vccnz L_slow_i0%=")
    o.label("L_join_i0")
    o.e(f"v_add_f32 v{LRUN}, v{LRUN}, v{LSUM}")

    # ---- two tile periods: t even (tp = 0), t odd (tp = 1) ---------------------------------------
    for tp in (0, 1):
        o.label(f"L_period{tp}")
        # odd iteration 2 t + 1: barrier of tile t, PV(2 t) from V(t) key steps 0, 1, S(2 t + 2) from K(t + 1) block 0
        # even iteration 2 t + 2: PV(2 t + 1) from V(t) key steps 2, 3, S(2 t + 3) from K(t + 1) block 1
        mask_block(o, 1, f"o{tp}")
        stamp(o)
        o.e("s_waitcnt vmcnt(0)")
        stamp(o)
        o.e("s_barrier")
        stamp(o)
        pairs = iteration_pairs(1, 1 - tp, 0, tp, 0) + iteration_pairs(0, 1 - tp, 1, tp, 2)
        chunks = spread(softmax_ops(1), 16) + spread(softmax_ops(0), 16)

        def between(tp=tp):
            o.e(f"s_cbranch_vccnz L_slow_o{tp}%=")
            o.label(f"L_join_o{tp}")
            o.e(f"v_add_f32 v{LRUN}, v{LRUN}, v{LSUM}")
            o.e(f"s_sub_u32 {S_NT}, {S_NT}, 1")
            o.e(f"s_cmp_eq_u32 {S_NT}, 0")
            o.e(f"s_cbranch_scc1 L_exit{tp}%=")
            mask_block(o, 0, f"e{tp}")

        # the requests go out behind the first fragment reads; stream() emits those first, so
        # the DMA block is hooked in front of pair 0
        stream(o, pairs, chunks, mid={0: (lambda tp=tp: dma_block(o, tp, f"p{tp}", paged)), 16: between})
        o.e(f"s_cbranch_vccnz L_slow_e{tp}%=")
        o.label(f"L_join_e{tp}")
        o.e(f"v_add_f32 v{LRUN}, v{LRUN}, v{LSUM}")
        if tp == 1:
            o.e("s_branch L_period0%=")

    # ---- exits: PV of the last block (bank 1, V(t) key steps 2 and 3) ------------------------------
    # The ring holds the first eight fragments of the even iteration: slots 1, 3, 5, 7 are
    # V(t) key step 2, blocks 0..3; slots 0, 2, 4, 6 (K fragments nobody needs) take key step 3.
    for tp in (0, 1):
        o.label(f"L_exit{tp}")
        o.e("s_waitcnt lgkmcnt(0)")
        for db in range(4):
            for x in frag_reads(("V", tp, 3, db), 2 * db):
                o.e(x)
        for db in range(4):
            o.e(mfma(("PV", db, 1, 0), 2 * db + 1))
        o.e("s_waitcnt lgkmcnt(0)")
        for db in range(4):
            o.e(mfma(("PV", db, 1, 1), 2 * db))
        o.e("s_branch L_end%=")

    slow_path(o, 0, "L_slow_i0", "L_join_i0")
    for tp in (0, 1):
        slow_path(o, 1, f"L_slow_o{tp}", f"L_join_o{tp}")
        slow_path(o, 0, f"L_slow_e{tp}", f"L_join_e{tp}")
    o.label("L_end")
    stamp(o)
    o.e("s_nop 15")
    o.e("s_nop 15")
    return o.lines


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else "/dev/stdout"
    with open(out, "w") as f:
        f.write("// Generated by gen_prefill_stream.py; do not edit.\n#pragma once\n")
        for name, paged in (("DENSE", False), ("PAGED", True)):
            f.write(f"#define TTPA_STREAM_LOOP_TEXT_{name} \\\n")
            for ln in generate(paged):
                f.write(f'  "{ln}\\n\\t" \\\n')
            f.write('  ""\n')
        regs = ", ".join([f'"v{r}"' for r in CLOBBERED] + [f'"{r}"' for r in SCALAR_CLOBBERS])
        f.write(f"#define TTPA_STREAM_LOOP_CLOBBERS {regs}\n")


if __name__ == "__main__":
    main()
