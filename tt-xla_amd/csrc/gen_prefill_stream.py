#!/usr/bin/env python3
"""Writes the hand-scheduled loop of the prefill kernel (head size 128, four query heads of one KV
head per workgroup, 32 query rows per wavefront, two workgroups per CU) as one block of gfx950
assembly per K / V source: build/prefill_stream_asm.h, included by prefill.hip.

Why assembly: the loop wants the matrix pipe and the vector ALU of a SIMD busy at the same time
from one instruction stream, with every register chosen by hand (256 per wavefront at two
wavefronts per SIMD) and every wait counted.  The unit of work is a BLOCK of 32 keys:

  S(i)   8 matrix instructions   S^T = K . Q^T of block i          (K fragments from LDS)
  sm(i)  ~56 vector instructions  p = exp2(s c - m), packed to bfloat16, row sum
  PV(i)  8 matrix instructions   O^T += V^T . P^T of block i       (V^T fragments from LDS)

Iteration i issues S(i + 1) and PV(i - 1) alternately, one slice of sm(i) and the LDS read of a
fragment 8 matrix instructions ahead behind each; the fragment reads run on across iterations.
Scores and probabilities alternate between two register banks by the parity of i, so nothing is
copied.

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

LDS: a ring of NS slots of 8 KiB (32 rows) for K blocks and one for V blocks; block j lives in
slot j % NS.  Iteration i reads K block i + 1 and V block i - 1 and, through the running fragment
reads, the first fragments of K block i + 2 and V block i.  Its barrier, at its start, says that
nobody reads K block i and V block i - 2 any more; K block i + NS and V block i + NS - 2 are
requested into their slots (LDS-DMA loads, two per tensor and wavefront).  A request has to have
landed NS - 2 barriers later: the wait in front of a barrier lets the requests of the last two
barriers stay in flight (vmcnt(8)), so a tile has three iterations to arrive with NS = 5, where
two stages of whole tiles gave it two.  Once requests have been skipped (no such block) the wait
is for everything.  Dense K / V: a block is `stride` bytes behind the one before.  Paged (block
size a multiple of 64): two blocks are a tile, a tile lies in one cache block; the table entry of
the tile K enters two iterations from now is requested in front of the tile requests of every
odd iteration (so the same wait covers it) and read at the next odd one.  Entries outside
[0, num_blocks) read cache block 0.

A workgroup takes one or several ITEMS (blocks of 32 query rows of its four heads) one after the
other: item k of the workgroup in slot j of `spg` slots is row block nqt - 1 - d with
d = k spg + (k even ? j : spg - 1 - j), as long as d < nqt.  Row blocks are dealt heavy first and in
alternating direction, so that with causal masking every workgroup gets about the same number of
key blocks.  The launcher's default is one item per workgroup (spg = nqt: the hardware deals the
workgroups as slots free up, which measured faster than one static round), several when the row
blocks weigh the same and divide evenly over one round.  Per item the block does everything
between the Q fragments and the stored output rows: its first requests (K blocks 0..NS-1, V blocks
0..NS-3; for the first item they are a block of assembly of their own, so that the caller's Q loads
overlap them), all blocks, the last PV, normalisation and store; then the next item's Q fragments
and first requests go out in front of the store of the finished one.

Matrix-to-vector hazards the hardware does not interlock are kept by construction: the vector
instructions that read a score bank start two matrix instructions after the last one that wrote
it (the mask waits explicitly); a bank of probabilities is rewritten three matrix instructions
after the last one that read it; the slow path and the exit wait out the matrix pipe with s_nop.
"""

import sys


# ---- register map (vector registers) ---------------------------------------------------------
ACC = [0, 16, 32, 48]          # output accumulators, head-dim blocks 0..3 (inputs / outputs)
QF = 64                        # Q fragments, k-step ks at QF + 4 ks (inputs)
S = [96, 112]                  # score banks
P = [128, 136]                 # probability banks (8 packed pairs each)
RING = 144                     # 8 fragment slots of 4 registers
NSLOT = 8
KOFF = 176                     # LDS byte address of the lane's K fragment in K slot 0, k-step ks (inputs)
VOFF = 184                     # ... of the lane's V^T fragment in V slot 0, output block db (inputs)
LDK = 188                      # per-lane global byte offsets of the 2 K loads of a block (inputs)
LDV = 190                      # ... of the 2 V loads
MC, LRUN, LSUM, ALPHA = 196, 197, 198, 199   # MC, LRUN: inputs / outputs
T = [200, 201, 202, 203]
ORV, MLOC, MB, MCN = 204, 205, 206, 207
PTREQ = 208                    # paged: the requested block-table entry (input)
LIMIT = 212                    # last visible key of the lane's row, minus 4 h (input)
LIMREL, NEGINF, VZERO = 213, 214, 215
QBASE, OUTBASE = 216, 218      # per lane, 64-bit: q / out of row 0 of the lane's head, at the lane's 8 h / 4 h elements (inputs)
VN, V4H = 220, 221             # lane % 32 and 4 (lane / 32) (inputs)
OUTP, PTMP, VT0, VROW = 222, 224, 226, 227
CLOBBERED = (list(range(0, QF)) + list(range(S[0], RING + 4 * NSLOT)) + list(range(MC, MCN + 1)) + [209, 210, 211, LIMIT, LIMREL, NEGINF, VZERO]
             + list(range(OUTP, VROW + 1)))

# ---- scalar registers ---------------------------------------------------------------------------
S_KBASE = "s[64:65]"           # dense: next K block to request; paged: the K cache (both minus 1024, see dma)
S_VBASE = "s[66:67]"
S_STRIDE = "s68"               # dense: bytes from one block to the next; paged: bytes of one (cache block, head) slab
S_C = "s69"                    # softmax scale times log2(e)
S_NB = "s70"                   # blocks left
S_KLEFT = "s71"                # K blocks left to request
S_M0B = "s72"                  # LDS address of this wavefront's first 1 KiB segment in K slot 0
S_VLEFT = "s73"                # V blocks left to request
S_MASKFROM = "s74"             # blocks whose first key is >= this are masked
S_KEY0 = "s75"                 # first key of the block whose softmax comes next
# paged only
S_HKV, S_HK, S_NCB, S_TPB = "s76", "s77", "s78", "s79"  # kv heads, this kv head, cache blocks, tiles per cache block
S_CIN = "s80"                  # tile-in-cache-block index of the tile whose entry is read next
S_RIN = "s81"                  # ... of the tile whose entry is requested next
S_RPTR = "s[82:83]"            # address of that entry
S_OFFV = "s[84:85]"            # byte offset in a cache of the tile V requests from (on entry: tile 1)
S_OFFK = "s[86:87]"            # ... K requests from (on entry: tile 2)
S_RLEFT = "s96"                # entries left to request
S_OFF0 = "s[98:99]"            # byte offset of tile 0
# items
S_K, S_J, S_SPG, S_NQT = "s40", "s41", "s42", "s43"      # item counter, slot of the workgroup, slots, row blocks
S_SQ, S_SKV, S_OFFSET, S_CAUSAL = "s44", "s45", "s46", "s47"
S_QTS, S_OTS = "s48", "s49"    # bytes from a query / output row to the next
# dense: s[50:51], s[52:53] K / V block 0 (minus 1024); paged: tile 1 and 2 offsets, s54 entry of tile 3,
# s55 / s56 tile-in-cache-block of tiles 3 / 4, s[58:59] address of tile 4's entry
S_ROW0 = "s57"                 # first query row of the item
S_STOREMASK = "s[60:61]"
# temporaries s[88:95], s[62:63]
SCALAR_CLOBBERS = [f"s{r}" for r in list(range(88, 96)) + [60, 61, 62, 63, 74, 75]]

NS = 5                         # slots per ring
UNROLL = 10                    # lcm(2, NS): score bank and slots repeat
SLOT = 8192
VRING = NS * SLOT              # LDS offset of the V ring; VOFF carries it
KEY_CONST = [8 * (r // 4) + r % 4 for r in range(16)]


class Out:
    def __init__(self):
        self.lines = []

    def e(self, s):
        self.lines.append(s)

    def label(self, name):
        self.lines.append(name + "%=:")


def vr(a, n=1):
    return f"v{a}" if n == 1 else f"v[{a}:{a + n - 1}]"


def frag_reads(frag, slot):
    """LDS read instructions of a fragment into ring slot `slot`.
    ("K", LDS slot, k-step) or ("V", LDS slot, key step 0 / 1, output block)."""
    base = RING + 4 * slot
    if frag[0] == "K":
        _, ls, ks = frag
        return [f"ds_read_b128 {vr(base, 4)}, v{KOFF + ks} offset:{ls * SLOT}"]
    _, ls, k4, db = frag
    off = ls * SLOT + k4 * 4096
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


def stream(o, pairs, valu_chunks, in_flight, tail):
    """pairs: [(matrix instruction, fragment)].  Per pair: wait for its fragment, the matrix
    instruction, the read of the fragment NSLOT pairs on, the vector chunk.  in_flight: the first
    NSLOT fragments have been requested by the code in front (else they are requested here);
    tail: the fragments requested behind the last NSLOT pairs (the next iteration's first ones)."""
    frags = [f for _, f in pairs] + list(tail)
    n = len(pairs)
    count = lambda f: len(frag_reads(frags[f], 0))
    if not in_flight:
        for f in range(min(NSLOT, len(frags))):
            for x in frag_reads(frags[f], f % NSLOT):
                o.e(x)
    for j in range(n):
        after = sum(count(f) for f in range(j + 1, min(j + NSLOT, len(frags))))
        assert after <= 15
        o.e(f"s_waitcnt lgkmcnt({after})")
        o.e(mfma(pairs[j][0], j % NSLOT))
        if j + NSLOT < len(frags):
            for x in frag_reads(frags[j + NSLOT], j % NSLOT):
                o.e(x)
        for x in valu_chunks[j]:
            o.e(x)


def iteration_pairs(p, has_pv=True):
    """Iteration i = p (mod UNROLL): S(i + 1) into bank 1 - q from K block i + 1, PV(i - 1) from
    bank 1 - q of the probabilities and V block i - 1."""
    q = p % 2
    pairs = []
    for x in range(8):
        pairs.append((("S", 1 - q, x), ("K", (p + 1) % NS, x)))
        if has_pv:
            pairs.append((("PV", x % 4, 1 - q, x // 4), ("V", (p - 1) % NS, x // 4, x % 4)))
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


def two_loads(o, lane_regs, base):
    """The instruction offset moves the LDS address as well as the global one: load j lands 1024 j
    bytes behind M0 and reads base + lane offset + 1024 j, so the lane offsets carry
    1024 - 1024 j and the bases - 1024."""
    for j in range(2):
        o.e(f"global_load_lds_dwordx4 v{lane_regs + j}, {base} offset:{1024 * j}")


def request_block(o, which, slot, tag, paged, half):
    """One K or V block into LDS slot `slot` of its ring, if there is one left to request.
    paged: the block is half `half` of the tile at S_OFFK / S_OFFV."""
    left, lane, base, ring = (S_KLEFT, LDK, S_KBASE, 0) if which == "K" else (S_VLEFT, LDV, S_VBASE, VRING)
    o.e(f"s_cmp_eq_u32 {left}, 0")
    o.e(f"s_cbranch_scc1 L_no{which}_{tag}%=")
    if paged:
        lo, hi = (86, 87) if which == "K" else (84, 85)
        b0 = int(base[2:4])
        o.e(f"s_add_u32 s90, s{b0}, s{lo}")
        o.e(f"s_addc_u32 s91, s{b0 + 1}, s{hi}")
        if half:
            o.e(f"s_add_u32 s90, s90, {SLOT}")
            o.e("s_addc_u32 s91, s91, 0")
    o.e(f"s_add_u32 m0, {S_M0B}, {ring + slot * SLOT}")
    o.e("s_nop 0")
    two_loads(o, lane, "s[90:91]" if paged else base)
    if not paged:
        b0 = int(base[2:4])
        o.e(f"s_add_u32 s{b0}, s{b0}, {S_STRIDE}")
        o.e(f"s_addc_u32 s{b0 + 1}, s{b0 + 1}, 0")
    o.e(f"s_sub_u32 {left}, {left}, 1")
    o.label(f"L_no{which}_{tag}")


def next_tile(o, tag):
    """paged, odd iterations: V moves on to the tile K was in, K to the tile whose entry has
    arrived; the entry after that is requested."""
    o.e("s_mov_b64 s[84:85], s[86:87]")
    o.e(f"v_readfirstlane_b32 s88, v{PTREQ}")
    o.e(f"s_cmp_lt_u32 s88, {S_NCB}")
    o.e("s_cselect_b32 s88, s88, 0")
    o.e(f"s_mul_i32 s88, s88, {S_HKV}")
    o.e(f"s_add_u32 s90, s88, {S_HK}")            # cache block * kv_heads + kv_head
    o.e(f"s_mul_hi_u32 s87, s90, {S_STRIDE}")
    o.e(f"s_mul_i32 s86, s90, {S_STRIDE}")
    o.e(f"s_lshl_b32 s90, {S_CIN}, 14")           # 64 tokens of 256 bytes per tile inside the cache block
    o.e("s_add_u32 s86, s86, s90")
    o.e("s_addc_u32 s87, s87, 0")
    o.e(f"s_add_u32 {S_CIN}, {S_CIN}, 1")
    o.e(f"s_cmp_eq_u32 {S_CIN}, {S_TPB}")
    o.e(f"s_cselect_b32 {S_CIN}, 0, {S_CIN}")
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


def iteration_head(o, p, tag, paged):
    """Mask, barrier and requests of iteration i = p (mod UNROLL)."""
    mask_block(o, p % 2, tag)
    # requests of the last two barriers may stay in flight, unless some were skipped
    o.e(f"s_cmp_eq_u32 {S_KLEFT}, 0")
    o.e(f"s_cbranch_scc1 L_all_{tag}%=")
    o.e("s_waitcnt vmcnt(8)")
    o.e(f"s_branch L_bar_{tag}%=")
    o.label(f"L_all_{tag}")
    o.e("s_waitcnt vmcnt(0)")
    o.label(f"L_bar_{tag}")
    o.e("s_barrier")
    if paged and p % 2 == 1:
        next_tile(o, tag)
    # K block i + NS is half (i + NS) % 2 of its tile, V block i + NS - 2 the same half of its own
    request_block(o, "K", p % NS, tag, paged, (p + NS) % 2)
    request_block(o, "V", (p + NS - 2) % NS, tag, paged, (p + NS) % 2)


def iteration_tail(o, tag, exit_label):
    o.e(f"s_cbranch_vccnz L_slow_{tag}%=")
    o.label(f"L_join_{tag}")
    o.e(f"v_add_f32 v{LRUN}, v{LRUN}, v{LSUM}")
    o.e(f"s_sub_u32 {S_NB}, {S_NB}, 1")
    o.e(f"s_cmp_eq_u32 {S_NB}, 0")
    o.e(f"s_cbranch_scc1 {exit_label}%=")


def first_frags(p):
    """The first NSLOT fragments of iteration p (mod UNROLL)."""
    return [f for _, f in iteration_pairs(p % UNROLL)[:NSLOT]]


def item_setup(o, tag):
    """Per-item state from S_ROW0: output pointers, the rows' key limits, the mask threshold, cleared
    accumulators and softmax state."""
    o.e(f"v_add_u32 v{VROW}, {S_ROW0}, v{VN}")                                   # the lane's query row
    o.e(f"v_mad_u64_u32 v[{OUTP}:{OUTP + 1}], s[92:93], v{VROW}, {S_OTS}, v[{OUTBASE}:{OUTBASE + 1}]")
    o.e(f"v_cmp_gt_i32_e64 {S_STOREMASK}, {S_SQ}, v{VROW}")                      # rows that exist are stored
    o.e(f"s_sub_u32 s88, {S_SQ}, 1")
    o.e(f"v_min_i32 v{VT0}, s88, v{VROW}")                                       # rows past the end repeat the last one
    o.e(f"v_add_u32 v{VT0}, {S_OFFSET}, v{VT0}")
    o.e(f"s_sub_u32 s89, {S_SKV}, 1")
    o.e(f"v_min_i32 v{VT0}, s89, v{VT0}")                                        # causal: min(offset + row, skv - 1)
    o.e(f"s_add_u32 s88, {S_OFFSET}, {S_ROW0}")
    o.e("s_min_i32 s88, s88, s89")
    o.e(f"s_cmp_eq_u32 {S_CAUSAL}, 0")
    o.e("s_cselect_b32 s88, s89, s88")                                           # the first row's limit
    o.e(f"s_cbranch_scc0 L_causal_{tag}%=")
    o.e(f"v_mov_b32 v{VT0}, s89")                                                # not causal: skv - 1 for every row
    o.label(f"L_causal_{tag}")
    o.e(f"v_sub_u32 v{LIMIT}, v{VT0}, v{V4H}")
    o.e(f"s_sub_u32 {S_MASKFROM}, s88, 30")
    o.e(f"s_mov_b32 {S_KEY0}, 0")
    o.e(f"v_mov_b32 v{MC}, 0xff800000")
    o.e(f"v_mov_b32 v{LRUN}, 0")
    for r in range(64):
        o.e(f"v_mov_b32 v{r}, 0")


def item_blocks(o):
    """S_NB / requests left from S_ROW0: the 32-key blocks any row of the item can see."""
    o.e(f"s_add_u32 s88, {S_ROW0}, 32")
    o.e(f"s_min_i32 s88, s88, {S_SQ}")
    o.e(f"s_add_u32 s88, s88, {S_OFFSET}")
    o.e(f"s_min_i32 s88, s88, {S_SKV}")
    o.e(f"s_cmp_eq_u32 {S_CAUSAL}, 0")
    o.e(f"s_cselect_b32 s88, {S_SKV}, s88")
    o.e("s_add_u32 s88, s88, 31")
    o.e(f"s_lshr_b32 {S_NB}, s88, 5")
    o.e(f"s_mov_b32 {S_KLEFT}, {S_NB}")
    o.e(f"s_mov_b32 {S_VLEFT}, {S_NB}")


def epilogue(o):
    """Normalises the item's accumulators and stores its rows: lane (n, h) holds, in accumulator
    register 16 db + 4 j + i, head-dim element 32 db + 8 j + 4 h + i of query row n.  The output pointer
    of lane (n, h) is row n's plus 16 h bytes."""
    o.e(f"v_mov_b32 v{MB}, v{LRUN}")
    o.e("s_nop 1")
    o.e(f"v_permlane32_swap_b32 v{LRUN}, v{MB}")
    o.e("s_nop 1")
    o.e(f"v_add_f32 v{ALPHA}, v{LRUN}, v{MB}")          # the row's sum: both halves of its keys
    o.e(f"v_rcp_f32 v{ALPHA}, v{ALPHA}")
    o.e("s_nop 1")
    for r in range(64):
        o.e(f"v_mul_f32 v{r}, v{ALPHA}, v{r}")
    for i in range(32):
        o.e(f"v_cvt_pk_bf16_f32 v{S[0] + i}, v{2 * i}, v{2 * i + 1}")
    o.e("s_nop 1")
    # The two lanes of a row trade halves, so that each stores 16 consecutive bytes (a row's 32 bytes per
    # instruction): lane (n, 0) keeps its block j and takes (n, 1)'s, lane (n, 1) ends with both blocks j + 1.
    for db in range(4):
        for jp in range(2):
            x = S[0] + 8 * db + 4 * jp
            o.e(f"v_permlane32_swap_b32 v{x}, v{x + 2}")
            o.e(f"v_permlane32_swap_b32 v{x + 1}, v{x + 3}")
    o.e("s_nop 3")
    o.e(f"s_and_saveexec_b64 s[62:63], {S_STOREMASK}")
    o.e("s_nop 1")
    for db in range(4):
        for jp in range(2):
            src = S[0] + 8 * db + 4 * jp
            o.e(f"global_store_dwordx4 v[{OUTP}:{OUTP + 1}], v[{src}:{src + 3}], off offset:{64 * db + 32 * jp} nt")   # written once, read by a later kernel
    o.e("s_mov_b64 exec, s[62:63]")
    o.e("s_nop 1")


def next_item(o, paged):
    """Behind the last PV of an item: is there another one?  Its Q fragments and first requests go
    out first, then the finished item is stored, then the state of the new one is set up."""
    o.e(f"s_add_u32 {S_K}, {S_K}, 1")
    o.e(f"s_mul_i32 s88, {S_K}, {S_SPG}")
    o.e(f"s_sub_u32 s89, {S_SPG}, 1")
    o.e(f"s_sub_u32 s89, s89, {S_J}")
    o.e(f"s_bitcmp1_b32 {S_K}, 0")
    o.e(f"s_cselect_b32 s89, s89, {S_J}")               # odd items are dealt in the other direction
    o.e("s_add_u32 s88, s88, s89")                      # d: the item's rank among the row blocks, heavy first
    o.e(f"s_cmp_ge_u32 s88, {S_NQT}")
    o.e("s_cbranch_scc1 L_last_item%=")
    o.e(f"s_sub_u32 s88, {S_NQT}, s88")
    o.e("s_sub_u32 s88, s88, 1")
    o.e(f"s_lshl_b32 {S_ROW0}, s88, 5")                 # (the finished item's pointers and store mask stay in registers)
    o.e("s_barrier")                                    # everybody has left the rings
    o.e(f"v_add_u32 v{VROW}, {S_ROW0}, v{VN}")
    o.e(f"s_sub_u32 s88, {S_SQ}, 1")
    o.e(f"v_min_i32 v{VROW}, s88, v{VROW}")
    o.e(f"v_mad_u64_u32 v[{PTMP}:{PTMP + 1}], s[92:93], v{VROW}, {S_QTS}, v[{QBASE}:{QBASE + 1}]")
    for ks in range(8):
        o.e(f"global_load_dwordx4 {vr(QF + 4 * ks, 4)}, v[{PTMP}:{PTMP + 1}], off offset:{32 * ks}")
    item_blocks(o)
    if paged:
        o.e("s_mov_b64 s[84:85], s[50:51]")
        o.e("s_mov_b64 s[86:87], s[52:53]")
        o.e(f"v_mov_b32 v{PTREQ}, s54")
        o.e(f"s_mov_b32 {S_CIN}, s55")
        o.e(f"s_mov_b32 {S_RIN}, s56")
        o.e("s_mov_b64 s[82:83], s[58:59]")
        o.e(f"s_sub_u32 s88, {S_NB}, 1")
        o.e("s_lshr_b32 s88, s88, 1")
        o.e("s_sub_u32 s88, s88, 3")
        o.e("s_max_i32 s88, s88, 0")
        o.e(f"s_mov_b32 {S_RLEFT}, s88")
    else:
        o.e("s_mov_b64 s[64:65], s[50:51]")
        o.e("s_mov_b64 s[66:67], s[52:53]")
    for ln in generate_first(paged, "nx"):
        o.lines.append(ln)
    epilogue(o)
    item_setup(o, "nx")
    o.e("s_branch L_item_top%=")
    o.label("L_last_item")
    epilogue(o)


def generate_first(paged, suffix=""):
    """The first requests: K blocks 0 .. NS - 1, V blocks 0 .. NS - 3 (a block of its own, so that
    the caller can put its Q loads behind them)."""
    o = Out()
    for j in range(NS):
        if paged:  # tiles 0, 1, 2 at S_OFF0, S_OFFV, S_OFFK
            src = ("s[98:99]", S_OFFV, S_OFFK)[j // 2]
            lo = int(src[2:4])
            o.e(f"s_cmp_eq_u32 {S_KLEFT}, 0")
            o.e(f"s_cbranch_scc1 L_noK_pro{j}{suffix}%=")
            o.e(f"s_add_u32 s90, s64, s{lo}")
            o.e(f"s_addc_u32 s91, s65, s{lo + 1}")
            if j % 2:
                o.e(f"s_add_u32 s90, s90, {SLOT}")
                o.e("s_addc_u32 s91, s91, 0")
            o.e(f"s_add_u32 m0, {S_M0B}, {j * SLOT}")
            o.e("s_nop 0")
            two_loads(o, LDK, "s[90:91]")
            o.e(f"s_sub_u32 {S_KLEFT}, {S_KLEFT}, 1")
            o.label(f"L_noK_pro{j}{suffix}")
        else:
            request_block(o, "K", j, f"pro{j}{suffix}", False, 0)
    for j in range(NS - 2):
        if paged:
            src = ("s[98:99]", S_OFFV)[j // 2]
            lo = int(src[2:4])
            o.e(f"s_cmp_eq_u32 {S_VLEFT}, 0")
            o.e(f"s_cbranch_scc1 L_noV_pro{j}{suffix}%=")
            o.e(f"s_add_u32 s90, s66, s{lo}")
            o.e(f"s_addc_u32 s91, s67, s{lo + 1}")
            if j % 2:
                o.e(f"s_add_u32 s90, s90, {SLOT}")
                o.e("s_addc_u32 s91, s91, 0")
            o.e(f"s_add_u32 m0, {S_M0B}, {VRING + j * SLOT}")
            o.e("s_nop 0")
            two_loads(o, LDV, "s[90:91]")
            o.e(f"s_sub_u32 {S_VLEFT}, {S_VLEFT}, 1")
            o.label(f"L_noV_pro{j}{suffix}")
        else:
            request_block(o, "V", j, f"pro{j}{suffix}", False, 0)
    return o.lines


def generate(paged):
    o = Out()
    assert NS == 5 and UNROLL == 10
    o.e(f"v_mov_b32 v{VZERO}, 0")
    item_setup(o, "first")
    o.label("L_item_top")
    o.e("s_waitcnt vmcnt(0)")
    o.e("s_barrier")
    # ---- S(0) from K block 0; behind it the fragments of iteration 0 (K block 1) ------------------
    pairs = [(("S", 0, x), ("K", 0, x)) for x in range(8)]
    it0 = iteration_pairs(0, has_pv=False)
    stream(o, pairs, [[] for _ in pairs], False, [f for _, f in it0])
    # ---- iteration 0: S(1), sm(0) ---------------------------------------------------------------
    o.e("s_nop 7")
    iteration_head(o, 0, "i0", paged)
    stream(o, it0, spread(softmax_ops(0), 8), True, first_frags(1))
    iteration_tail(o, "i0", "L_exit0")
    # ---- iterations 1 .. : ten in a row, then round again -------------------------------------------
    for k in range(UNROLL):
        p = (k + 1) % UNROLL
        o.label(f"L_it{p}")
        iteration_head(o, p, f"p{p}", paged)
        stream(o, iteration_pairs(p), spread(softmax_ops(p % 2), 16), True, first_frags(p + 1))
        iteration_tail(o, f"p{p}", f"L_exit{p}")
    o.e("s_branch L_it1%=")

    # ---- exits: PV of the last block i = p (mod UNROLL) -----------------------------------------------
    # The ring holds the first eight fragments of the iteration that is not coming: slots 1, 3, 5, 7
    # are V block i, key step 0, output blocks 0..3; slots 0, 2, 4, 6 (K fragments nobody needs) take
    # key step 1.
    for p in range(UNROLL):
        o.label(f"L_exit{p}")
        o.e("s_waitcnt lgkmcnt(0)")
        for db in range(4):
            for x in frag_reads(("V", p % NS, 1, db), 2 * db):
                o.e(x)
        for db in range(4):
            o.e(mfma(("PV", db, p % 2, 0), 2 * db + 1))
        o.e("s_waitcnt lgkmcnt(0)")
        for db in range(4):
            o.e(mfma(("PV", db, p % 2, 1), 2 * db))
        o.e("s_branch L_end%=")

    slow_path(o, 0, "L_slow_i0", "L_join_i0")
    for p in range(UNROLL):
        slow_path(o, p % 2, f"L_slow_p{p}", f"L_join_p{p}")
    o.label("L_end")
    o.e("s_nop 15")
    o.e("s_nop 15")
    next_item(o, paged)
    return o.lines


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else "/dev/stdout"
    with open(out, "w") as f:
        f.write("// Generated by gen_prefill_stream.py; do not edit.\n#pragma once\n")
        for name, paged in (("DENSE", False), ("PAGED", True)):
            for macro, lines in ((f"TTPA_STREAM_FIRST_TEXT_{name}", generate_first(paged)),
                                 (f"TTPA_STREAM_LOOP_TEXT_{name}", generate(paged))):
                f.write(f"#define {macro} \\\n")
                for ln in lines:
                    f.write(f'  "{ln}\\n\\t" \\\n')
                f.write('  ""\n')
        regs = ", ".join([f'"v{r}"' for r in CLOBBERED] + [f'"{r}"' for r in SCALAR_CLOBBERS])
        f.write(f"#define TTPA_STREAM_LOOP_CLOBBERS {regs}\n")
        f.write(f"#define TTPA_STREAM_LDS_BYTES {2 * NS * SLOT}\n#define TTPA_STREAM_V_RING {VRING}\n")


if __name__ == "__main__":
    main()
