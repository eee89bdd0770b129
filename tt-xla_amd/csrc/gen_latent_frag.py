#!/usr/bin/env python3
"""Writes the matrix-instruction sequences of the latent attention kernels that share K in LDS
(decode_wide.hip: latent_prefill_kernel, paged_decode_latent128_kernel) as blocks of gfx950 assembly:
build/latent_frag_asm.h.

A wavefront has a SIMD to itself and owns two blocks of 16 rows.  Per step of 32 keys (two 16-row
pieces of K in LDS) it computes, for each row block,
  S^T = K . Q^T        2 x DQK / 32 v_mfma_f32_16x16x32_bf16, A = a K fragment (ds_read_b128)
  O^T += V^T . P^T     DV / 16 v_mfma_f32_16x16x32_bf16, A = the V^T fragments of the two pieces
                       (two ds_read_b64_tr_b16), K dimension = the 32 keys
and every fragment read feeds the matrix instructions of both row blocks: with one block of rows per
wavefront the four SIMDs of a CU would ask LDS for 4 x 1 KiB per 16 cycles, all it delivers.

Why assembly.  Written as C++ with a ring of prefetched fragments, the compiler folds the ring into
one register set and waits for every read right before the matrix instruction that uses it; and a
wavefront that is alone on its SIMD has nobody to fill the vector unit and the address path while
its matrix instructions run, so the softmax of the next step's scores and the LDS-DMA requests for
a later step are placed between the matrix instructions here.  Registers are fixed:

  a[0:2 DV/4)         O^T accumulators, DV / 4 per row block, 4 per block of 16 value columns
  v[0:2 DQK/8)        Q fragments, DQK / 8 per row block, 4 per step of 32 features
  then                a ring of 5 fragments (4 registers: a K fragment or a pair of V^T fragments),
                      the four score tiles (16), softmax temporaries (8), the next step's probabilities
                      (8)

Two row blocks of (576, 512) fill all 256 accumulation registers, more than the compiler binds to
the operands of one assembly statement, so no variable stands for the accumulators: the blocks below
are the only code that names an accumulation register (check_latent_frag.py checks the compiled
kernels for that), every one of them lists all 256 as clobbered, and volatile statements keep their
order.  Everything else (LDS addresses of the lane's fragments, probabilities) comes in registers
that the compiler chooses.

A step without masks is one statement (whole_step): its two products share one pipeline of fragment
reads, so the second one starts on fragments that were requested while the first one ran.  The
products also exist on their own (scores, values) for steps whose softmax is C++ (masks).

A ring slot is refilled one matrix instruction after the last one that read it.  Waits are counted: a
block starts with lgkmcnt(0), so the counter holds its own reads only.  Matrix results are read by
vector instructions no earlier than 16 wait states after the last matrix instruction (s_nop at the
end of a block), and a block's first matrix instruction comes two wait states behind the vector
instructions that wrote its operands.

The chunk index of a row is swizzled inside aligned groups of GC chunks (Latent16::position), so a
lane has GC / 4 (K) or GC / 2 (V^T) base addresses and the group is an immediate offset; the second
piece of a step lies 32 DQK bytes behind the first.
"""
import sys

RB = 2
DEPTH = 5
# (head size, value width, chunks per swizzle group)
SHAPES = ((576, 512, 8), (576, 384, 8), (192, 128, 8), (128, 128, 16))

# Lines that bracket every block which names an accumulation register
MARK_BEGIN, MARK_END = "; latent-frag accumulators begin", "; latent-frag accumulators end"
ACC_CLOBBERS = [f'"a{r}"' for r in range(256)]


class Regs:
    def __init__(self, dqk, dv):
        self.nq, self.nacc = dqk // 8, dv // 4  # registers of one row block's Q / accumulators
        self.ring = RB * self.nq
        self.st = self.ring + 4 * DEPTH
        self.tmp = self.st + 8 * RB
        self.pn = self.tmp + 4 * RB
        self.ml = self.pn + 4 * RB
        assert RB * self.nacc <= 256 and self.ml + 2 * RB <= 208

    def q(self, b, s):
        r = self.nq * b + 4 * s
        return f"v[{r}:{r + 3}]"

    def slot(self, i, lo=0, n=4):
        r = self.ring + 4 * i + lo
        return f"v[{r}:{r + n - 1}]"

    def score(self, b, pc):
        r = self.st + 8 * b + 4 * pc
        return f"v[{r}:{r + 3}]"

    def accum(self, b, j):
        r = self.nacc * b + 4 * j
        return f"a[{r}:{r + 3}]"

    def ring_clobbers(self):
        return [f'"v{r}"' for r in range(self.ring, self.ring + 4 * DEPTH)]


def pipeline(n, read, mma, covers, after_fill=()):
    """n steps; read(j, slot) returns the read instructions of step j into ring slot `slot` = j % depth,
    mma(j, slot) the matrix instructions that use them.  The slot of step j - 1 is refilled behind the
    first matrix instruction of step j.  covers(j): the last step whose reads the wait in front of step
    j covers, or None for no wait there (a wavefront alone on its SIMD issues one instruction per four
    cycles, whatever the kind: a wait is not free).  after_fill: lines behind the reads that fill the
    ring at the start."""
    depth = min(DEPTH, n)
    lines, queue = [], []  # queue: (step, read instructions) in the order of issue

    def issue(j):
        r = read(j, j % depth)
        queue.append((j, len(r)))
        return r

    for j in range(depth):
        lines += issue(j)
    lines += list(after_fill)
    waited = -1
    for j in range(n):
        last = covers(j)
        if last is not None:
            at = [k for k, (step, _) in enumerate(queue) if step == last]
            assert len(at) == 1 and last >= j, "a wait covers reads that are under way"
            behind = sum(c for _, c in queue[at[0] + 1:])
            assert behind <= 15
            lines.append(f"s_waitcnt lgkmcnt({behind})")
            waited = last
        assert waited >= j
        ops = mma(j, j % depth)
        lines.append(ops[0])
        nxt = j - 1 + depth
        if j >= 1 and nxt < n:
            lines += issue(nxt)
        lines += ops[1:]
    assert [step for step, _ in queue] == list(range(n))
    return lines


def every(k, n):
    """covers() of pipeline: a wait in front of every k-th of n steps."""
    return lambda j: min(j + k - 1, n - 1) if j % k == 0 else None


def spread(lines, extra, first=1, last_fraction=1.0):
    """Puts the instruction groups `extra` behind matrix instructions of `lines`: the first group behind
    matrix instruction number `first`, the last behind number `last_fraction` x their count, the others
    evenly between."""
    n_mma = sum(1 for ln in lines if ln.startswith("v_mfma"))
    last = max(int(n_mma * last_fraction), first)
    where = [first + (u * (last - first)) // max(len(extra) - 1, 1) for u in range(len(extra))]
    out, seen, used = [], 0, 0
    for ln in lines:
        out.append(ln)
        if ln.startswith("v_mfma"):
            seen += 1
            while used < len(extra) and where[used] <= seen:
                out += extra[used]
                used += 1
    assert used == len(extra)
    return out


def asm_body(lines):
    return " \\\n".join(f'      "{ln}\\n\\t"' for ln in lines)


def statement(comment, name, args, lines, outs, ins, clob):
    return f"""{comment}
__device__ __forceinline__ void {name}({", ".join(args)}) {{
  asm volatile(
{asm_body(lines)}
      : {", ".join(outs)}
      : {", ".join(ins)}
      : {", ".join(clob + ['"memory"'])});
}}
"""


def q_operands(R, dqk):
    nq16, rem = divmod(dqk // 32, 4)
    assert rem in (0, 2) and nq16 >= 1
    args, ins = [], []
    for b in range(RB):
        base = R.nq * b
        args += [f"const u32x16 &q{b}_{i}" for i in range(nq16)]
        ins += [f'"{{v[{base + 16 * i}:{base + 16 * i + 15}]}}"(q{b}_{i})' for i in range(nq16)]
        if rem:
            args.append(f"const u32x8 &q{b}_{nq16}")
            ins.append(f'"{{v[{base + 16 * nq16}:{base + 16 * nq16 + 7}]}}"(q{b}_{nq16})')
    return args, ins


def scores(dqk, dv, gc, requests=0, nt=False):
    """Both pieces of a step, their steps of 32 features alternating (four independent accumulation
    chains).  requests > 0: with the wavefront's LDS-DMA requests for a later step between the matrix
    instructions (request_groups)."""
    R = Regs(dqk, dv)
    ksteps, piece, kb = dqk // 32, 32 * dqk, gc // 4
    n_out = 2 * RB

    def where(j):
        return j % 2, j // 2  # piece, step of 32 features

    def read(j, slot):
        pc, s = where(j)
        return [f"ds_read_b128 {R.slot(slot)}, %{n_out + s % kb} offset:{pc * piece + 16 * gc * (s // kb)}"]

    def mma(j, slot):
        pc, s = where(j)
        return [f"v_mfma_f32_16x16x32_bf16 {R.score(b, pc)}, {R.slot(slot)}, {R.q(b, s)}, {'0' if s == 0 else R.score(b, pc)}"
                for b in range(RB)]

    lines = ["s_waitcnt lgkmcnt(0)"] + pipeline(2 * ksteps, read, mma, every(1, 2 * ksteps)) + ["s_nop 7", "s_nop 7"]
    args = [f"floatx4 &st{2 * b + pc}" for b in range(RB) for pc in range(2)] + [f"uint32_t kb{i}" for i in range(kb)]
    outs = [f'"=&{{{R.score(b, pc)}}}"(st{2 * b + pc})' for b in range(RB) for pc in range(2)]
    ins = [f'"v"(kb{i})' for i in range(kb)]
    qa, qi = q_operands(R, dqk)
    args, ins = args + qa, ins + qi
    clob, name = R.ring_clobbers(), f"latent_scores_{dqk}"
    if requests:
        first = len(outs) + len(ins)
        off, base, dst = first, first + requests, first + requests + 4
        args += [f"uint32_t off{j}" for j in range(requests)] + [f"const void *base{i}" for i in range(4)] + ["uint32_t dst"]
        ins += [f'"v"(off{j})' for j in range(requests)] + [f'"s"(base{i})' for i in range(4)] + ['"s"(dst)']
        assert len(outs) + len(ins) <= 30
        req = request_groups(requests, off, base, dst, nt)
        lines = spread(lines, req, first=4, last_fraction=0.75)
        clob, name = clob + ['"m0"', '"scc"'], name + "_req" + ("_nt" if nt else "")
    comment = (f"// S^T = K . Q^T of the two pieces of a step: {ksteps} steps of 32 features, swizzle groups of {gc} chunks" +
               (f"\n// (with {requests} LDS-DMA requests{', non-temporal,' if nt else ''} between the matrix instructions)" if requests else ""))
    return statement(comment, name, args, lines, outs, ins, clob)


def values_pipeline(R, dv, gc, piece, pf_in, vb_in):
    vbases = gc // 2

    def read(j, slot):
        base, off = f"%{vb_in + j % vbases}", 16 * gc * (j // vbases)
        return [f"ds_read_b64_tr_b16 {R.slot(slot, 0, 2)}, {base} offset:{off}",
                f"ds_read_b64_tr_b16 {R.slot(slot, 2, 2)}, {base} offset:{off + piece}"]

    def mma(j, slot):
        return [f"v_mfma_f32_16x16x32_bf16 {R.accum(b, j)}, {R.slot(slot)}, %{pf_in + b}, {R.accum(b, j)}" for b in range(RB)]

    return pipeline(dv // 16, read, mma, every(1, dv // 16))


def values(dqk, dv, gc):
    R = Regs(dqk, dv)
    vbases = gc // 2
    lines = ([MARK_BEGIN, "s_nop 1", "s_waitcnt lgkmcnt(0)"] + values_pipeline(R, dv, gc, 32 * dqk, 0, RB) +
             ["s_nop 7", "s_nop 7", MARK_END])
    args = [f"const u32x4 &pf{b}" for b in range(RB)] + [f"uint32_t vb{i}" for i in range(vbases)]
    ins = [f'"v"(pf{b})' for b in range(RB)] + [f'"v"(vb{i})' for i in range(vbases)]
    return statement(f"// O^T += V^T . P^T of a step: {dv // 16} blocks of 16 value columns, swizzle groups of {gc} chunks",
                     f"latent_values_{dqk}_{dv}", args, lines, [], ins, R.ring_clobbers() + ACC_CLOBBERS)


def softmax_groups(R, scale, m, th, total, moved):
    """Softmax of the score tiles of one step against the running maxima as they are, without masks:
    per row block b the 8 scores of a lane (R.st + 8 b .., left as they are), the running maximum in
    operand m + b, the probabilities exp2(score * scale - maximum) as bfloat16 pairs in R.pn + 4 b ..
    and their sum (taken before rounding) in operand total + b.  A maximum moves only when a score
    exceeds it by more than 8 (as in the C++ form): operand th + b holds (maximum + 8) / scale, and
    the scalar pair `moved` collects the lanes with a raw score above it; the caller redoes the
    softmax of a step where any lane has one.  `scale` is positive.
    Returns groups of instructions that stay together; the two row blocks alternate group by group, so
    that neighbours do not depend on each other (a wavefront issues in order: a vector instruction
    that waits holds up the matrix instruction behind it)."""
    phases = []
    for b in range(RB):
        S = [f"v{R.st + 8 * b + k}" for k in range(8)]
        T = [f"v{R.tmp + 4 * b + k}" for k in range(4)]
        P = [f"v{R.pn + 4 * b + k}" for k in range(4)]
        M, TH, SUM = f"%{m + b}", f"%{th + b}", f"%{total + b}"
        g = [[f"v_max3_f32 {T[0]}, {S[0]}, {S[1]}, {S[2]}"], [f"v_max3_f32 {T[0]}, {T[0]}, {S[3]}, {S[4]}"],
             [f"v_max3_f32 {T[0]}, {T[0]}, {S[5]}, {S[6]}"], [f"v_max_f32 {T[0]}, {T[0]}, {S[7]}"],
             [f"v_cmp_gt_f32 vcc, {T[0]}, {TH}", f"s_or_b64 {moved}, {moved}, vcc"]]
        for k in range(4):
            x, y = (T[1], T[2]) if k % 2 == 0 else (T[3], T[0])  # (two pairs of temporaries in turn; the maximum is done with)
            g += [[f"v_fma_f32 {x}, {S[2 * k]}, {scale}, -{M}"], [f"v_fma_f32 {y}, {S[2 * k + 1]}, {scale}, -{M}"],
                  [f"v_exp_f32 {x}, {x}"], [f"v_exp_f32 {y}, {y}"],
                  [f"v_add_f32 {SUM}, {x}, {y}"] if k == 0 else [f"v_add_f32 {SUM}, {SUM}, {x}"]]
            if k:
                g += [[f"v_add_f32 {SUM}, {SUM}, {y}"]]
            g += [[f"v_cvt_pk_bf16_f32 {P[k]}, {x}, {y}"]]
        phases.append(g)
    out = []
    for groups in zip(*phases):
        out += list(groups)
    return out


def request_groups(requests, off, base, dst, nt):
    """The wavefront's LDS-DMA requests for a later step (a 1 KiB request occupies the address path for
    16 cycles, and a wavefront that waits for it issues nothing else): request j reads 16 bytes per
    lane at base (j % 4) + offset j and lands at LDS address dst + 1024 j (base i = the step's address
    - 1024 i: the instruction offset 1024 i moves the LDS address and the global address alike, so
    four requests share a value of M0).  off, base, dst: the first operand numbers."""
    req = []
    for j in range(requests):
        r = []
        if j % 4 == 0:
            r += [f"s_mov_b32 m0, %{dst}" if j == 0 else f"s_add_u32 m0, %{dst}, {1024 * j}", "s_nop 0"]
        r.append(f"global_load_lds_dwordx4 %{off + j}, %{base + j % 4}" + (f" offset:{1024 * (j % 4)}" if j % 4 else "") +
                 (" nt" if nt else ""))
        req.append(r)
    return req


def whole_step(dqk, dv, gc, requests=0, nt=False):
    """A step as one statement and one pipeline, the workgroup's barrier included (the caller has
    waited for its own requests): the score product of the step at kb.., then the second
    product of the step before (at vb.., probabilities pf) with the softmax of the new scores between
    its matrix instructions.  The ring slots that the last score steps leave take the first V^T
    fragments, so the matrix unit goes from one product to the other without a gap (as two statements
    the second one starts with reads of its own and their latency: a twentieth of a step)."""
    R = Regs(dqk, dv)
    ksteps, piece, kb, vbases = dqk // 32, 32 * dqk, gc // 4, gc // 2
    ns, nv = 2 * ksteps, dv // 16
    # operands: outputs 0..3 score tiles, 4..5 next probabilities, 6..7 their sums, 8 the lanes whose
    # maximum has to move; inputs: K bases, V^T bases, Q, maxima, thresholds, probabilities, scale, (requests)
    n_out = 4 * RB + 1
    st_out, pn_out, sum_out, moved = 0, 2 * RB, 3 * RB, f"%{4 * RB}"
    kb_in = n_out
    vb_in = kb_in + kb
    qa, qi = q_operands(R, dqk)
    m_in = vb_in + vbases + len(qi)
    th_in, pf_in = m_in + RB, m_in + 2 * RB
    scale = f"%{pf_in + RB}"

    # The statement starts with the workgroup's barrier of the step (behind it the step's K is in LDS).
    # The step before has been there since the barrier before, so where the second product is long enough
    # its first `early` blocks go first: their reads go out in front of the barrier and their matrix
    # instructions run while the first K fragments are on their way.
    early = DEPTH if nv >= 4 * DEPTH else 0
    order = [("v", t) for t in range(early)] + [("s", k) for k in range(ns)] + [("v", t) for t in range(early, nv)]

    def read(j, slot):
        kind, t = order[j]
        if kind == "s":
            pc, f = t % 2, t // 2  # piece, step of 32 features
            return [f"ds_read_b128 {R.slot(slot)}, %{kb_in + f % kb} offset:{pc * piece + 16 * gc * (f // kb)}"]
        base, off = f"%{vb_in + t % vbases}", 16 * gc * (t // vbases)
        return [f"ds_read_b64_tr_b16 {R.slot(slot, 0, 2)}, {base} offset:{off}",
                f"ds_read_b64_tr_b16 {R.slot(slot, 2, 2)}, {base} offset:{off + piece}"]

    def mma(j, slot):
        kind, t = order[j]
        if kind == "s":
            pc, f = t % 2, t // 2
            return [f"v_mfma_f32_16x16x32_bf16 {R.score(b, pc)}, {R.slot(slot)}, {R.q(b, f)}, {'0' if f == 0 else R.score(b, pc)}"
                    for b in range(RB)]
        return [f"v_mfma_f32_16x16x32_bf16 {R.accum(b, t)}, {R.slot(slot)}, %{pf_in + b}, {R.accum(b, t)}" for b in range(RB)]

    def covers(j):  # every step up to the last score step, then every second one
        late = j - early - ns
        if late < 0:
            return j
        return min(j + 1, ns + nv - 1) if late % 2 == 0 else None

    if early:
        assert early == DEPTH  # (the reads that fill the ring are those of the step before)
        lines = pipeline(ns + nv, read, mma, covers, after_fill=["s_barrier"])
    else:
        lines = ["s_barrier"] + pipeline(ns + nv, read, mma, covers)
    split = 1 + max(k for k, ln in enumerate(lines) if ln.startswith("v_mfma") and " a[" not in ln)
    first, second = lines[:split], lines[split:]
    # the vector unit reads the score tiles no earlier than 16 wait states behind their last matrix instruction
    count = seen = 0
    for ln in second:
        count += 1
        seen += ln.startswith("v_mfma")
        if count >= 16:
            break
    assert count >= 16 and seen + 1 < 2 * (nv - early)
    second = spread(second, softmax_groups(R, scale, m_in, th_in, sum_out, moved), first=seen + 1)
    args = ([f"floatx4 &st{2 * b + pc}" for b in range(RB) for pc in range(2)] + [f"u32x4 &pn{b}" for b in range(RB)] +
            [f"float &sum{b}" for b in range(RB)] + ["uint64_t &moved"] + [f"uint32_t kb{i}" for i in range(kb)] +
            [f"uint32_t vb{i}" for i in range(vbases)] + qa + [f"float m{b}" for b in range(RB)] + [f"float th{b}" for b in range(RB)] +
            [f"const u32x4 &pf{b}" for b in range(RB)] + ["float scale"])
    outs = ([f'"=&{{{R.score(b, pc)}}}"(st{2 * b + pc})' for b in range(RB) for pc in range(2)] +
            [f'"=&{{v[{R.pn + 4 * b}:{R.pn + 4 * b + 3}]}}"(pn{b})' for b in range(RB)] + [f'"=&v"(sum{b})' for b in range(RB)] + ['"=&s"(moved)'])
    ins = ([f'"v"(kb{i})' for i in range(kb)] + [f'"v"(vb{i})' for i in range(vbases)] + qi + [f'"v"(m{b})' for b in range(RB)] +
           [f'"v"(th{b})' for b in range(RB)] + [f'"v"(pf{b})' for b in range(RB)] + ['"s"(scale)'])
    assert len(outs) == n_out and R.score(0, 0) == f"v[{R.st}:{R.st + 3}]"
    clob = R.ring_clobbers() + [f'"v{r}"' for r in range(R.tmp, R.tmp + 4 * RB)] + ['"vcc"', '"scc"']
    name = f"latent_step_{dqk}_{dv}"
    if requests:
        at = len(outs) + len(ins)
        args += [f"uint32_t off{j}" for j in range(requests)] + [f"const void *base{i}" for i in range(4)] + ["uint32_t dst"]
        ins += [f'"v"(off{j})' for j in range(requests)] + [f'"s"(base{i})' for i in range(4)] + ['"s"(dst)']
        first = spread(first, request_groups(requests, at, at + requests, at + requests + 4, nt), first=4, last_fraction=0.75)
        clob, name = clob + ['"m0"'], name + "_req" + ("_nt" if nt else "")
    lines = ([MARK_BEGIN, f"s_mov_b64 {moved}, 0", "s_nop 0", "s_waitcnt lgkmcnt(0)"] + first + second + ["s_nop 7", "s_nop 7", MARK_END])
    comment = (f"// One step, from the workgroup's barrier on: S^T = K . Q^T of the two pieces at kb.. ({ksteps} steps of 32 features), then O^T += V^T . P^T of the step\n"
               f"// at vb.. ({nv} blocks of 16 value columns, probabilities pf) and, between its matrix instructions, the softmax of\n"
               "// the new score tiles st.. against the running maxima m.. as they are (no masks, scale > 0): pn the\n"
               "// probabilities, sum their sums, moved != 0 where a score exceeds th = (m + 8) / scale" +
               (f"\n// (with {requests} LDS-DMA requests{', non-temporal,' if nt else ''} between the matrix instructions of the first product)"
                if requests else ""))
    return statement(comment.replace("\\n", "\n"), name, args, lines, outs, ins, clob + ACC_CLOBBERS)


def accumulator_access(dv):
    nacc = dv // 4
    out = []
    clear = [MARK_BEGIN] + [f"v_accvgpr_write_b32 a{r}, 0" for r in range(RB * nacc)] + [MARK_END]
    out.append(statement("// all accumulators = 0", f"latent_acc_clear_{dv}", [], clear, [], [], ACC_CLOBBERS))
    # the 16 accumulators of four blocks of 16 value columns: f[4 j + r] = value 16 (4 i + j) + 4 quad + r
    for b in range(RB):
        for i in range(nacc // 16):
            base = nacc * b + 16 * i
            rd = [MARK_BEGIN] + [f"v_accvgpr_read_b32 %{r}, a{base + r}" for r in range(16)] + [MARK_END]
            out.append(statement("", f"latent_acc_read_{dv}_{b}_{i}", ["float (&f)[16]"], rd, [f'"=v"(f[{r}])' for r in range(16)], [], []))
    return "\n".join(out)


def accumulator_scale(dqk, dv):
    R = Regs(dqk, dv)
    scale = [MARK_BEGIN]
    for b in range(RB):
        for r0 in range(0, R.nacc, 8):
            regs = [(R.nacc * b + r0 + i, R.ring + i) for i in range(8)]
            scale += [f"v_accvgpr_read_b32 v{v}, a{a}" for a, v in regs]
            scale += [f"v_mul_f32 v{v}, v{v}, %{b}" for a, v in regs]
            scale += [f"v_accvgpr_write_b32 a{a}, v{v}" for a, v in regs]
    scale += [MARK_END]
    return statement("// accumulators of row block b *= alpha b (through the ring registers)", f"latent_acc_scale_{dqk}_{dv}",
                     [f"float alpha{b}" for b in range(RB)], scale, [], [f'"v"(alpha{b})' for b in range(RB)],
                     R.ring_clobbers() + ACC_CLOBBERS)


def wrappers(dqk, dv, gc, requests):
    """struct LatentBlocks<DQK, DV>: the blocks of one shape behind one set of names."""
    R = Regs(dqk, dv)
    ksteps, kb, vbases = dqk // 32, gc // 4, gc // 2
    nq16, rem = divmod(ksteps, 4)
    per = R.nacc // 16
    qs = ", ".join(", ".join([f"q16[{b}][{i}]" for i in range(nq16)] + ([f"q8[{b}]"] if rem else [])) for b in range(RB))
    st = ", ".join(f"st[{b}][{pc}]" for b in range(RB) for pc in range(2))
    kf = ", ".join(f"step + kf[{i}]" for i in range(kb))
    vf = ", ".join(f"step + vf[{i}]" for i in range(vbases))
    vp = ", ".join(f"before + vf[{i}]" for i in range(vbases))
    offs = ", ".join(f"off[{j}]" for j in range(requests))
    reads = "\n".join(f"    {'if' if k == 0 else 'else if'} constexpr (B == {k // per} && I == {k % per}) latent_acc_read_{dv}_{k // per}_{k % per}(f);"
                      for k in range(RB * per))
    return f"""template <>
struct LatentBlocks<{dqk}, {dv}> {{
  static constexpr int REQUESTS = {requests};  // LDS-DMA requests of a wavefront per step
  static __device__ __forceinline__ void scores(uint32_t step, floatx4 (&st)[2][2], const uint32_t (&kf)[{kb}], const u32x16 (&q16)[2][{nq16}],
                                                const u32x8 (&q8)[2]) {{
    latent_scores_{dqk}({st}, {kf}, {qs});
  }}
  template <bool STREAMING>
  static __device__ __forceinline__ void scores_requesting(uint32_t step, floatx4 (&st)[2][2], const uint32_t (&kf)[{kb}],
                                                           const u32x16 (&q16)[2][{nq16}], const u32x8 (&q8)[2],
                                                           const uint32_t (&off)[{requests}], const char *from, uint32_t dst) {{
    if constexpr (STREAMING)
      latent_scores_{dqk}_req_nt({st}, {kf}, {qs}, {offs}, from, from - 1024, from - 2048, from - 3072, dst);
    else
      latent_scores_{dqk}_req({st}, {kf}, {qs}, {offs}, from, from - 1024, from - 2048, from - 3072, dst);
  }}
  static __device__ __forceinline__ void values(uint32_t step, const u32x4 (&pf)[2], const uint32_t (&vf)[{vbases}]) {{
    latent_values_{dqk}_{dv}(pf[0], pf[1], {vf});
  }}
  // (`before`: the step whose second product this is)
  static __device__ __forceinline__ void whole_step(uint32_t step, uint32_t before, floatx4 (&st)[2][2], u32x4 (&pn)[2], float (&sum)[2],
                                                    uint64_t &moved, const uint32_t (&kf)[{kb}], const uint32_t (&vf)[{vbases}],
                                                    const u32x16 (&q16)[2][{nq16}], const u32x8 (&q8)[2], const float (&m)[2],
                                                    const float (&th)[2], const u32x4 (&pf)[2], float scale) {{
    latent_step_{dqk}_{dv}({st}, pn[0], pn[1], sum[0], sum[1], moved, {kf}, {vp}, {qs}, m[0], m[1], th[0], th[1], pf[0], pf[1], scale);
  }}
  template <bool STREAMING>
  static __device__ __forceinline__ void whole_step_requesting(uint32_t step, uint32_t before, floatx4 (&st)[2][2], u32x4 (&pn)[2],
                                                               float (&sum)[2], uint64_t &moved, const uint32_t (&kf)[{kb}],
                                                               const uint32_t (&vf)[{vbases}], const u32x16 (&q16)[2][{nq16}],
                                                               const u32x8 (&q8)[2], const float (&m)[2], const float (&th)[2],
                                                               const u32x4 (&pf)[2], float scale, const uint32_t (&off)[{requests}],
                                                               const char *from, uint32_t dst) {{
    if constexpr (STREAMING)
      latent_step_{dqk}_{dv}_req_nt({st}, pn[0], pn[1], sum[0], sum[1], moved, {kf}, {vp}, {qs}, m[0], m[1], th[0], th[1], pf[0], pf[1], scale,
                                    {offs}, from, from - 1024, from - 2048, from - 3072, dst);
    else
      latent_step_{dqk}_{dv}_req({st}, pn[0], pn[1], sum[0], sum[1], moved, {kf}, {vp}, {qs}, m[0], m[1], th[0], th[1], pf[0], pf[1], scale,
                                 {offs}, from, from - 1024, from - 2048, from - 3072, dst);
  }}
  static __device__ __forceinline__ void clear() {{ latent_acc_clear_{dv}(); }}
  static __device__ __forceinline__ void scale(float alpha0, float alpha1) {{ latent_acc_scale_{dqk}_{dv}(alpha0, alpha1); }}
  template <int B, int I>
  static __device__ __forceinline__ void read16(float (&f)[16]) {{
{reads}
  }}
}};
"""


def main():
    out = sys.argv[1] if len(sys.argv) > 1 else "/dev/stdout"
    with open(out, "w") as f:
        f.write("// Generated by gen_latent_frag.py; do not edit.\n#pragma once\n\n")
        f.write("template <int DQK, int DV>\nstruct LatentBlocks;\n\n")
        done = set()

        def once(key, text):
            if key not in done:
                done.add(key)
                f.write(text + "\n")

        for dqk, dv, gc in SHAPES:
            requests = 2 * (32 * dqk // 1024) // 4  # a step's 16-byte-per-lane requests, a quarter per wavefront
            once(("scores", dqk), scores(dqk, dv, gc))
            once(("req", dqk), scores(dqk, dv, gc, requests=requests))
            once(("req_nt", dqk), scores(dqk, dv, gc, requests=requests, nt=True))
            f.write(values(dqk, dv, gc) + "\n")
            f.write(whole_step(dqk, dv, gc) + "\n")
            f.write(whole_step(dqk, dv, gc, requests=requests) + "\n")
            f.write(whole_step(dqk, dv, gc, requests=requests, nt=True) + "\n")
            once(("acc", dv), accumulator_access(dv))
            f.write(accumulator_scale(dqk, dv) + "\n")
            f.write(wrappers(dqk, dv, gc, requests) + "\n")


if __name__ == "__main__":
    main()
