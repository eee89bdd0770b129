"""The assembly blocks that csrc/gen_latent_frag.py writes for the latent kernels, executed on a model
of what the hardware guarantees (no GPU): LDS reads return in order and `s_waitcnt lgkmcnt(N)` leaves
at most the N youngest under way; a matrix instruction must find its fragment landed, a ring slot may be
refilled only behind every matrix instruction that reads it, the vector unit may read a score tile no
earlier than 16 wait states behind its last matrix instruction.  On top of the ordering rules the model
checks the mathematics of a block: every (row block, piece, feature step) of the score product and
every (row block, value block) of the second product exactly once and on the right fragment, and the
softmax between the matrix instructions against a direct evaluation."""

import importlib.util
import math
import pathlib
import random
import re
import struct

import pytest

CSRC = pathlib.Path(__file__).resolve().parents[1] / "tt-xla_amd" / "csrc"
_spec = importlib.util.spec_from_file_location("gen_latent_frag", CSRC / "gen_latent_frag.py")
G = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(G)

RB = G.RB


def _bf16(x):
    """float -> bfloat16 (round to nearest even) -> float"""
    bits = struct.unpack("<I", struct.pack("<f", x))[0]
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return struct.unpack("<f", struct.pack("<I", bits))[0]


def _parse(text):
    """-> (instructions, operand names in the order of their numbers, {name: pinned register range})"""
    body = text[text.index("asm volatile(") :]
    lines = re.findall(r'^\s+"(.*?)\\n\\t"', body, flags=re.M)
    tails = [ln for ln in body.splitlines() if ln.startswith("      : ")]
    assert len(tails) == 3
    names, pinned = [], {}
    for ln in tails[:2]:
        for constraint, name in re.findall(r'"([^"]*)"\(([^)]*)\)', ln):
            names.append(name)
            m = re.search(r"\{v\[(\d+):(\d+)\]\}", constraint)
            if m:
                pinned[name] = (int(m.group(1)), int(m.group(2)))
    return lines, names, pinned


def _vregs(tok):
    m = re.fullmatch(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return list(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.fullmatch(r"v(\d+)", tok)
    return [int(m.group(1))] if m else None


def run_block(text, dqk, dv, gc, want_scores, want_values, seed=0):
    lines, names, pinned = _parse(text)
    R = G.Regs(dqk, dv)
    ksteps, piece, nkb, nvb = dqk // 32, 32 * dqk, gc // 4, gc // 2
    ring = set(range(R.ring, R.ring + 4 * G.DEPTH))
    st_regs = set(range(R.st, R.st + 8 * RB))

    def opname(tok):
        m = re.fullmatch(r"-?%(\d+)", tok)
        return names[int(m.group(1))] if m else None

    rnd = random.Random(seed)
    scale = 0.7
    val = {}  # values of one lane: registers ("v123") and operands (by name)
    for b in range(RB):
        val[f"m{b}"] = rnd.uniform(-1.0, 1.0)
        val[f"th{b}"] = (val[f"m{b}"] + 8.0) / scale
    val["scale"] = scale
    for r in st_regs:
        val[f"v{r}"] = rnd.uniform(-4.0, 4.0)
    scores_in = {r: val[f"v{r}"] for r in st_regs}

    content = {}   # ring register -> (fragment id, part)
    readers = {}   # fragment id -> matrix instructions that have read it
    queue = []     # LDS reads under way, oldest first: (fragment id, registers)
    landed = set()
    since_reader = {}  # fragment id -> matrix instructions issued behind its last reader
    done_s, done_v = {}, {}
    barrier_at = last_score_mma = first_score_valu = None
    k_reads_before_barrier = 0
    slots = 0  # wait states issued so far
    moved = None

    def get(tok):
        neg = tok.startswith("-")
        tok = tok.lstrip("-")
        name = opname(tok)
        v = val[name] if name else val[tok]
        return -v if neg else v

    def put(tok, v):
        name = opname(tok)
        val[name if name else tok] = v

    for ln in lines:
        if ln.startswith(";"):
            continue
        op, _, rest = ln.partition(" ")
        args = [a.strip() for a in re.split(r",\s*(?![^\[]*\])", rest)] if rest else []
        here = slots
        slots += int(args[0]) + 1 if op == "s_nop" else 1
        if op == "s_waitcnt":
            n = int(re.fullmatch(r"lgkmcnt\((\d+)\)", args[0]).group(1))
            while len(queue) > n:
                landed.add(queue.pop(0)[0])
        elif op in ("ds_read_b128", "ds_read_b64_tr_b16"):
            dst = _vregs(args[0])
            base, off = opname(args[1].split()[0]), int(re.search(r"offset:(\d+)", ln).group(1))
            assert set(dst) <= ring and len(dst) == (4 if op == "ds_read_b128" else 2)
            frag = (op, base, off, here)
            for r in dst:
                if r in content:  # the fragment that the read replaces has served every reader
                    old = content[r][0]
                    assert readers.get(old, 0) == RB, f"{ln}: overwrites a fragment that {readers.get(old, 0)} of {RB} have read"
                    assert since_reader[old] >= 1, f"{ln}: right behind the last reader of its slot"
            for i, r in enumerate(dst):
                content[r] = (frag, i)
            queue.append((frag, dst))
            readers[frag] = 0
            if op == "ds_read_b128" and barrier_at is None:
                k_reads_before_barrier += 1
        elif op == "s_barrier":
            assert barrier_at is None
            barrier_at = here
        elif op == "v_mfma_f32_16x16x32_bf16":
            d, a, b_, c = args
            a_regs = _vregs(a)
            assert a_regs and set(a_regs) <= ring and len(a_regs) == 4
            frags = [content[r] for r in a_regs]
            for f, _ in frags:
                assert f in landed, f"{ln}: fragment {f[:3]} not waited for"
            for f in since_reader:
                since_reader[f] += 1
            for f in {f for f, _ in frags}:
                readers[f] += 1
                since_reader[f] = 0
            if d.startswith("a["):
                lo = int(re.fullmatch(r"a\[(\d+):(\d+)\]", d).group(1))
                blk, t = lo // R.nacc, (lo % R.nacc) // 4
                assert d == R.accum(blk, t) == c and opname(b_) == f"pf{blk}"
                (f0, i0), (f1, i1), (f2, i2), (f3, i3) = frags
                assert f0 == f1 and f2 == f3 and (i0, i1, i2, i3) == (0, 1, 0, 1)
                want_base, want_off = f"vb{t % nvb}", 16 * gc * (t // nvb)
                assert f0[:3] == ("ds_read_b64_tr_b16", want_base, want_off), (ln, f0)
                assert f2[:3] == ("ds_read_b64_tr_b16", want_base, want_off + piece), (ln, f2)
                assert (blk, t) not in done_v
                done_v[(blk, t)] = True
            else:
                d_regs, q_regs = _vregs(d), _vregs(b_)
                blk, f = q_regs[0] // R.nq, (q_regs[0] % R.nq) // 4
                pc = (d_regs[0] - R.st - 8 * blk) // 4
                assert b_ == R.q(blk, f) and d == R.score(blk, pc) and pc in (0, 1)
                assert c == ("0" if f == 0 else d), ln
                assert len({fr for fr, _ in frags}) == 1 and [i for _, i in frags] == [0, 1, 2, 3]
                assert frags[0][0][:3] == ("ds_read_b128", f"kb{f % nkb}", pc * piece + 16 * gc * (f // nkb)), (ln, frags[0][0])
                seen = done_s.setdefault((blk, pc), [])
                assert f == len(seen), f"{ln}: feature steps of a tile in order (the first one clears it)"
                seen.append(f)
                last_score_mma = here
        elif op == "global_load_lds_dwordx4":
            assert barrier_at is not None or "latent_step" not in text, "a request in front of the step's barrier"
        elif op in ("s_mov_b32", "s_add_u32"):
            assert args[0] == "m0"
        elif op == "s_mov_b64":
            assert args[1] == "0"
            moved = False
        elif op == "s_or_b64":
            assert args[0] == args[1] and args[2] == "vcc"
            moved = moved or val["vcc"]
        elif op == "s_nop":
            pass
        else:  # the softmax: one lane's arithmetic
            srcs = args[1:]
            if first_score_valu is None and any((_vregs(s.lstrip("-")) or [None])[0] in st_regs for s in srcs):
                first_score_valu = here
            x = [get(s) for s in srcs]
            if op == "v_max3_f32":
                put(args[0], max(x))
            elif op == "v_max_f32":
                put(args[0], max(x))
            elif op == "v_cmp_gt_f32":
                assert args[0] == "vcc"
                val["vcc"] = x[0] > x[1]
            elif op == "v_fma_f32":
                put(args[0], x[0] * x[1] + x[2])
            elif op == "v_exp_f32":
                put(args[0], 2.0 ** x[0])
            elif op == "v_add_f32":
                put(args[0], x[0] + x[1])
            elif op == "v_cvt_pk_bf16_f32":
                put(args[0], (_bf16(x[0]), _bf16(x[1])))
            else:
                raise AssertionError(f"unknown instruction: {ln}")

    assert all(n == RB for n in readers.values()), "every fragment that was read is used by both row blocks"
    if want_scores:
        assert sorted(done_s) == [(b, pc) for b in range(RB) for pc in range(2)]
        assert all(v == list(range(ksteps)) for v in done_s.values())
    else:
        assert not done_s
    if want_values:
        assert sorted(done_v) == [(b, t) for b in range(RB) for t in range(dv // 16)]
    else:
        assert not done_v
    if first_score_valu is not None:
        assert last_score_mma is None or first_score_valu - last_score_mma >= 16 + 1, (last_score_mma, first_score_valu)
        # probabilities, sums and the lanes whose maximum would move
        any_moved = False
        for b in range(RB):
            s = [scores_in[R.st + 8 * b + k] for k in range(8)]
            m = val[f"m{b}"]
            p = [2.0 ** (x * scale - m) for x in s]
            lo, hi = pinned[f"pn{b}"]
            for k in range(4):
                got = val[f"v{lo + k}"]
                assert got == (_bf16(p[2 * k]), _bf16(p[2 * k + 1])), (b, k, got)
            assert math.isclose(val[f"sum{b}"], sum(p), rel_tol=1e-12)
            any_moved = any_moved or max(s) > val[f"th{b}"]
        assert moved == any_moved
    return dict(barrier_at=barrier_at, k_reads_before_barrier=k_reads_before_barrier, tail=slots - 1 - (last_score_mma or 0),
                softmax=first_score_valu is not None)


@pytest.mark.parametrize("dqk,dv,gc", G.SHAPES)
def test_separate_products(dqk, dv, gc):
    requests = 2 * (32 * dqk // 1024) // 4
    for text in (G.scores(dqk, dv, gc), G.scores(dqk, dv, gc, requests=requests), G.scores(dqk, dv, gc, requests=requests, nt=True)):
        info = run_block(text, dqk, dv, gc, want_scores=True, want_values=False)
        assert info["barrier_at"] is None
        assert info["tail"] >= 16, "the compiler's code may read the score tiles right behind the block"
    run_block(G.values(dqk, dv, gc), dqk, dv, gc, want_scores=False, want_values=True)


@pytest.mark.parametrize("dqk,dv,gc", G.SHAPES)
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_whole_step(dqk, dv, gc, seed):
    requests = 2 * (32 * dqk // 1024) // 4
    for kw in ({}, {"requests": requests}, {"requests": requests, "nt": True}):
        text = G.whole_step(dqk, dv, gc, **kw)
        info = run_block(text, dqk, dv, gc, want_scores=True, want_values=True, seed=seed)
        assert info["barrier_at"] is not None, "the statement carries the step's barrier"
        assert info["k_reads_before_barrier"] == 0, "K of the step is in LDS only behind the barrier"
        assert info["softmax"]
        assert text.count("global_load_lds_dwordx4") == kw.get("requests", 0)


def test_the_model_notices_a_missing_wait_and_an_early_refill():
    dqk, dv, gc = G.SHAPES[0]
    text = G.whole_step(dqk, dv, gc)
    broken = text.replace('"s_waitcnt lgkmcnt(3)\\n\\t"', '"s_waitcnt lgkmcnt(4)\\n\\t"', 1)
    assert broken != text
    with pytest.raises(AssertionError, match="not waited for"):
        run_block(broken, dqk, dv, gc, True, True)
    lines = text.splitlines()
    k = next(i for i, ln in enumerate(lines) if "ds_read_b128" in ln)
    prev_mma = max(i for i in range(k) if "v_mfma" in lines[i])
    lines.insert(prev_mma, lines.pop(k))  # the first K read moves in front of the matrix instruction before it
    with pytest.raises(AssertionError, match="overwrites a fragment|right behind the last reader"):
        run_block("\n".join(lines), dqk, dv, gc, True, True)
