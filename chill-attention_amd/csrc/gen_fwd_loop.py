#!/usr/bin/env python3
"""Generates the hand-scheduled inner loop of the forward kernel (chill_fwd_fast.h) as an inline-asm
statement: chill_fwd_loop.inc, one macro per (element type, head dim, waves, stages).

Why generated assembly: the loop is bound by what a wave issues besides its MFMAs, and the order and
the registers of every instruction matter.  The generator lays the loop out in SLOTS of one MFMA each,
deals the softmax and the LDS reads over the slots, computes every s_waitcnt from the order of the LDS
reads, and checks the stream against the gfx950 hazards the compiler would otherwise take care of
(check_stream below).  It fails, and the build with it, if a check does not hold.

The statement works through `cnt` >= 1 whole 64-key tiles of predicate-free blocks, from the ring
rotation in front of the first one to the last O^T += V^T P^T:

    fill                          S(g), S(g+1) and P(g) of the first tile; V operands of step g
    while cnt > 1:  step 0, step 1, cnt -= 1, ring_top
    drain                         the two steps of the last tile without looking ahead
ring_top = wait for the tile ahead, barrier, rotate the ring, issue a new tile.  The caller does the
first one except for the issue.  While tiles remain to be issued, the scalar work of ring_top rides in
the slots of the steps (the loads of the tile under step 0, the rotation under step 1) and only the
wait and the barrier stand between two tiles.

Step g of the loop (parity PAR = g & 1), 2 * NS slots (NS = D / 16):
  matrix pipe   slots 0 .. NS-1:   O^T[db] += V(g)^T P(g)^T
                slots NS .. 2NS-1: S(g+2)^T = K(g+2) Q^T - m0   (the chain starts from `mneg`)
  vector ALU    P(g+1) = exp2(S(g+1)) -> packed pairs, row sum += P; nothing in slot 0 (S(g+1) is still
                settling in the matrix pipe)
  LDS           slot t < NS: K operand t of step g+2; slot NS + t: V operand t of step g+1, each into
                the registers of the operand the slot's MFMA has just taken
Register roles by parity: S[PAR] receives the new scores, S[PAR^1] is exponentiated; P[PAR] feeds the
matrix pipe, P[PAR^1] is written.
"""
from __future__ import annotations

import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from asm_stream import (MFMA_RESULT_WAIT, TRANS_USE_WAIT, VALU_TO_MFMA_WAIT, Stream, check_clobbers, check_stream,  # noqa: F401
                        rng, vr)

STAGE_PAD_K = 16   # bytes per K row beyond the data (PaddedTile, rowwise_pad)
STAGE_PAD_V = 64   # bytes per V row beyond the data (transposed_pad, rows of at least 128 bytes)

# the two tile pointers live in fixed scalar register pairs (their halves are added to separately)
PTR_SGPR = {"kb": 96, "vb": 98}
ABLATE_WAITS = False   # timing experiments that drop LDS reads wait for everything instead of counting


class Config:
    def __init__(self, elem: str, D: int, waves: int, stages: int, ablate=()):
        assert elem in ("bf16", "f16") and D in (64, 128) and stages in (3, 4)
        self.elem, self.D, self.NW, self.NSTG = elem, D, waves, stages
        self.ablate = set(ablate)         # timing experiments only: parts of the loop left out
        self.DB = D // 32
        self.NS = D // 16                 # slots (MFMAs) per phase; also operands per phase
        self.rb = D * 2
        self.kpitch = self.rb + STAGE_PAD_K
        self.vpitch = self.rb + STAGE_PAD_V
        self.kbytes = 64 * self.kpitch
        self.vbytes = 64 * self.vpitch
        self.stage = self.kbytes + self.vbytes
        self.kslabs = self.kbytes // 1024
        self.vslabs = self.vbytes // 1024
        assert self.kbytes % 1024 == 0 and self.vbytes % 1024 == 0
        self.FL = stages - 3              # tiles in flight beyond the certified one
        self.loads_min = self.kslabs // waves + self.vslabs // waves
        # register map
        r = 0
        self.O = r; r += 16 * self.DB
        self.Q = r; r += 4 * self.NS
        self.MNEG = r; r += 16
        self.S = (r, r + 16); r += 32
        self.P = (r, r + 8); r += 16
        # One set of operand registers serves both phases: the MFMA of slot t takes operand t, and the
        # LDS read issued right behind it refills the same registers with the operand of the other
        # phase (an MFMA has read its A and B operands long before an LDS read issued after it returns).
        self.OP = r; r += 4 * self.NS
        self.T = r; r += 4                # exp2 results in flight
        self.L = r; r += 1
        self.KLANE = r; r += 1
        self.VLANE = r; r += 1
        self.kper = (self.kslabs + waves - 1) // waves
        self.vper = (self.vslabs + waves - 1) // waves
        self.GK = r; r += self.kper
        self.GV = r; r += self.vper
        self.KA = r; r += 1               # K read address (next tile)
        self.VA = (r, r + 1); r += 2      # V read addresses (this tile, next tile)
        self.PSUM = r; r += 1             # f16: sum of P of the current block
        self.nvgpr = r
        self.mfma = "v_mfma_f32_32x32x16_" + elem
        self.cvt = "v_cvt_pk_bf16_f32" if elem == "bf16" else "v_cvt_pk_f16_f32"
        self.name = f"CHILL_FWD_LOOP_{elem.upper()}_{D}_{waves}_{stages}"


def softmax_ops(c: Config, st: Stream, s_in: int, p_out: int):
    """P = exp2(S) of one 32 x 32 block, packed, and its sum: a list of closures in issue order.
    (v_dot2c_f32_bf16 with a register of ones would sum two packed entries per instruction; measured,
    it is slower than the two additions it replaces.)"""
    ops = []
    acc = c.PSUM if c.elem == "f16" else c.L

    def exp(e):
        t = c.T + e % 4
        return lambda: st.add(f"v_exp_f32 {vr(t)}, {vr(s_in + e)}", "trans", [s_in + e], [t])

    def cvt(k):
        t0, t1 = c.T + (2 * k) % 4, c.T + (2 * k + 1) % 4
        d = p_out + k
        return lambda: st.add(f"{c.cvt} {vr(d)}, {vr(t0)}, {vr(t1)}", "valu", [t0, t1], [d])

    def add(e):
        t = c.T + e % 4
        if e == 0 and c.elem == "f16":
            return lambda: st.add(f"v_mov_b32 {vr(acc)}, {vr(t)}", "valu", [t], [acc])
        return lambda: st.add(f"v_add_f32 {vr(acc)}, {vr(acc)}, {vr(t)}", "valu", [acc, t], [acc])

    # the pack and the sums of a pair run behind the exponentials of the next pair (a v_exp_f32 result
    # needs a wait state before a vector instruction reads it)
    for k in range(8):
        ops += [exp(2 * k), exp(2 * k + 1)]
        if k > 0:
            ops += [cvt(k - 1), add(2 * k - 2), add(2 * k - 1)]
    ops += [cvt(7), add(14), add(15)]
    if "valu" in c.ablate:
        return []
    return ops


RAISE_ROW_SUM = "0x53800000"   # 2^40: a row sum above it has the reference raised (bf16; P and the sum reach 2^127)


def block_sum_check(c: Config, st: Stream, par: int, tag: str, tile_end: bool = True):
    """End of a step whose vector work has produced P[par ^ 1] from S[par ^ 1] (and, in the loop, whose matrix work
    has left the scores after those in S[par]): the row sums, and the test that sends the wave to `gen_raise`.
    fp16: every P of a block stays below 65504 while the lane's sum over the block stays below `blockhi`, tested after
    every block; bf16: the row sum is tested once per tile.  The branch is taken by the whole wave if any row asks."""
    if "valu" in c.ablate:
        return
    if c.elem == "f16":
        st.add(f"v_add_f32 {vr(c.L)}, {vr(c.L)}, {vr(c.PSUM)}", "valu", [c.L, c.PSUM], [c.L])
        st.add(f"v_cmp_lt_f32 vcc, %[blockhi], {vr(c.PSUM)}", "valu", [c.PSUM], [])
    elif tile_end:
        st.add(f"v_cmp_lt_f32 vcc, {RAISE_ROW_SUM}, {vr(c.L)}", "valu", [c.L], [])
    else:
        return
    st.ins.append(dict(text=f"s_cbranch_vccnz .Lraise{tag}%=", kind="raise", reads=set(), writes=set(), nops=1, lds=False,
                       wait=None, par=par, tag=tag))
    st.add(f".Lback{tag}%=:", "label", nops=0)


def gen_raise(c: Config, st: Stream, par: int):
    """The reference of the rows is raised by d = the largest exponent among the scores at hand (never lowered):
    S[par ^ 1] (whose P is packed in P[par ^ 1] and not yet part of O^T) and S[par]; the scores at hand, the start
    value of the score chains, O^T and the row sum follow, and P[par ^ 1] is computed again.  O^T and LSE2 do not
    depend on the reference beyond rounding (the running max of chill_fwd.py:188-286 does the same, block by block).
    Rare: the block is out of line."""
    A = st.add
    ripe, fresh, P = c.S[par ^ 1], c.S[par], c.P[par ^ 1]
    d, t0, t1, t2 = c.PSUM, c.T, c.T + 1, c.T + 2
    # what the matrix pipe may still be working on: the scores in `fresh`, O^T
    A("s_nop 7", "nop", nops=8)
    A("s_nop 7", "nop", nops=8)
    regs = rng(ripe, 16) + rng(fresh, 16)
    A(f"v_max3_f32 {vr(t0)}, {vr(regs[0])}, {vr(regs[1])}, {vr(regs[2])}", "valu", regs[:3], [t0])
    rest = regs[3:]
    while len(rest) >= 2:
        A(f"v_max3_f32 {vr(t0)}, {vr(t0)}, {vr(rest[0])}, {vr(rest[1])}", "valu", [t0] + rest[:2], [t0])
        rest = rest[2:]
    if rest:
        A(f"v_max_f32 {vr(t0)}, {vr(t0)}, {vr(rest[0])}", "valu", [t0, rest[0]], [t0])
    # the two lanes of a row (l and l ^ 32) hold half of its keys each and share its reference
    A(f"v_mov_b32 {vr(t1)}, {vr(t0)}", "valu", [t0], [t1])
    A("s_nop 1", "nop", nops=2)
    A(f"v_permlane32_swap_b32 {vr(t0)}, {vr(t1)}", "valu", [t0, t1], [t0, t1])
    A(f"v_max_f32 {vr(d)}, {vr(t0)}, {vr(t1)}", "valu", [t0, t1], [d])
    A(f"v_max_f32 {vr(d)}, 0, {vr(d)}", "valu", [d], [d])
    for r in regs + rng(c.MNEG, 16):
        A(f"v_sub_f32 {vr(r)}, {vr(r)}, {vr(d)}", "valu", [r, d], [r])
    A(f"v_exp_f32 {vr(t2)}, -{vr(d)}", "trans", [d], [t2])
    A("s_nop 0", "nop")
    A(f"v_mul_f32 {vr(c.L)}, {vr(c.L)}, {vr(t2)}", "valu", [c.L, t2], [c.L])
    for r in rng(c.O, 16 * c.DB):
        A(f"v_mul_f32 {vr(r)}, {vr(r)}, {vr(t2)}", "valu", [r, t2], [r])
    # P again, against the new reference (its share of the row sum has been scaled with the sum)
    pend = None
    for k in range(8):
        ta, tb = c.T + (2 * k) % 4, c.T + (2 * k + 1) % 4
        A(f"v_exp_f32 {vr(ta)}, {vr(ripe + 2 * k)}", "trans", [ripe + 2 * k], [ta])
        A(f"v_exp_f32 {vr(tb)}, {vr(ripe + 2 * k + 1)}", "trans", [ripe + 2 * k + 1], [tb])
        if pend is not None:
            A(*pend[:2], pend[2], pend[3])
        pend = (f"{c.cvt} {vr(P + k)}, {vr(ta)}, {vr(tb)}", "valu", [ta, tb], [P + k])
    A("s_nop 0", "nop")
    A(*pend[:2], pend[2], pend[3])
    A("s_nop 1", "nop", nops=2)


def mfma_pv(c: Config, st: Stream, t: int, p_in: int):
    s2, db = divmod(t, c.DB)
    o, a, b = c.O + 16 * db, c.OP + 4 * t, p_in + 4 * s2
    if "mfma" in c.ablate:
        return
    st.add(f"{c.mfma} {vr(o, 16)}, {vr(a, 4)}, {vr(b, 4)}, {vr(o, 16)}", "mfma", rng(a, 4) + rng(b, 4) + rng(o, 16),
           rng(o, 16))


def mfma_qk(c: Config, st: Stream, t: int, s_out: int):
    a, b = c.OP + 4 * t, c.Q + 4 * t
    cin = c.MNEG if t == 0 else s_out
    if "mfma" in c.ablate:
        return
    st.add(f"{c.mfma} {vr(s_out, 16)}, {vr(a, 4)}, {vr(b, 4)}, {vr(cin, 16)}", "mfma",
           rng(a, 4) + rng(b, 4) + rng(cin, 16), rng(s_out, 16))


def read_k(c: Config, st: Stream, t: int, addr: int, kb: int):
    d = c.OP + 4 * t
    if "lds" in c.ablate or "kread" in c.ablate:
        return
    st.add(f"ds_read_b128 {vr(d, 4)}, {vr(addr)} offset:{kb * 32 * c.kpitch + t * 32}", "lds", [addr], rng(d, 4), lds=True)


def read_v(c: Config, st: Stream, t: int, addr: int, kb: int):
    s2, db = divmod(t, c.DB)
    d = c.OP + 4 * t
    off = kb * 32 * c.vpitch + 16 * s2 * c.vpitch + db * 64
    if "lds" in c.ablate or "vread" in c.ablate:
        return
    if "vb128" in c.ablate:
        st.add(f"ds_read_b128 {vr(d, 4)}, {vr(c.KA)} offset:{off}", "lds", [addr], rng(d, 4), lds=True)
        return
    st.add(f"ds_read_b64_tr_b16 {vr(d, 2)}, {vr(addr)} offset:{off}", "lds", [addr], rng(d, 2), lds=True)
    st.add(f"ds_read_b64_tr_b16 {vr(d + 2, 2)}, {vr(addr)} offset:{off + 8 * c.vpitch}", "lds", [addr],
           rng(d + 2, 2), lds=True)


def wait_lgkm(st: Stream, n: int):
    if ABLATE_WAITS:
        n = 0
    st.add(f"s_waitcnt lgkmcnt({n})", "wait", wait=n)


def gen_step(c: Config, st: Stream, par: int, filler=(), late_filler=(), tag=""):
    """One step.  `filler`: closures (scalar work: ring rotation, tile loads) dealt over all slots;
    `late_filler`: closures dealt over the slots of the second phase only."""
    NS = c.NS
    ops = softmax_ops(c, st, c.S[par ^ 1], c.P[par ^ 1])
    nslots = 2 * NS
    # deal the vector work over slots 1 .. 2NS-1
    share = [0] * nslots
    for t in range(1, nslots):
        share[t] = len(ops) * t // (nslots - 1) - len(ops) * (t - 1) // (nslots - 1)
    fshare = [len(filler) * (t + 1) // nslots - len(filler) * t // nslots for t in range(nslots)]
    lshare = [0] * NS + [len(late_filler) * (t + 1) // NS - len(late_filler) * t // NS for t in range(NS)]
    it, fit, lit = iter(ops), iter(filler), iter(late_filler)

    def fill_slot(t):
        for _ in range(share[t]):
            next(it)()
        for _ in range(fshare[t]):
            next(fit)()
        for _ in range(lshare[t]):
            next(lit)()

    for t in range(NS):
        # LDS reads issued after V operand t: V t+1 .. NS-1 (2 each), then K 0 .. t-1
        wait_lgkm(st, 2 * (NS - 1 - t) + t)
        mfma_pv(c, st, t, c.P[par])
        read_k(c, st, t, c.KA, par)                       # K of step g+2: block `par` of the next tile
        fill_slot(t)
    for t in range(NS):
        # LDS reads issued after K operand t: K t+1 .. NS-1, then V 0 .. t-1 (2 each)
        wait_lgkm(st, (NS - 1 - t) + 2 * t)
        mfma_qk(c, st, t, c.S[par])
        # V of step g+1: block 1 of this tile (par = 0) or block 0 of the next (par = 1)
        read_v(c, st, t, c.VA[par], par ^ 1)
        fill_slot(NS + t)
    assert next(it, None) is None and next(fit, None) is None and next(lit, None) is None
    block_sum_check(c, st, par, tag + str(par), tile_end=(par == 1))


def issue_ops(c: Config, st: Stream):
    """The loads of one tile into the stage at `tfill` (tm0 = tfill + wave * 1024), as closures of one
    load each: K slabs j * NW + wave, then V slabs.  A wave without a slab in the last round runs that
    load with an empty EXEC (no branches: these closures are dealt over the slots of a step)."""
    ops = []
    A = st.add
    for kind, per, slabs, base, gbase, ptr in (("k", c.kper, c.kslabs, 0, c.GK, "kb"),
                                              ("v", c.vper, c.vslabs, c.kbytes, c.GV, "vb")):
        for j in range(per):
            partial = (j + 1) * c.NW > slabs

            def load(j=j, partial=partial, base=base, gbase=gbase, ptr=ptr, kind=kind):
                if partial:
                    A(f"s_mov_b64 exec, %[{kind}last]", "salu")
                A(f"s_add_u32 m0, %[tm0], {base + j * c.NW * 1024}", "salu")
                A("s_nop 0", "nop")
                A(f"global_load_lds_dwordx4 {vr(gbase + j)}, s[{PTR_SGPR[ptr]}:{PTR_SGPR[ptr] + 1}]", "vmem", [gbase + j])
                if partial:
                    A("s_mov_b64 exec, %[execsave]", "salu")
            ops.append(load)
        lo, hi = f"s{PTR_SGPR[ptr]}", f"s{PTR_SGPR[ptr] + 1}"

        def advance(lo=lo, hi=hi, kind=kind):
            A(f"s_add_u32 {lo}, {lo}, %[{kind}step]", "salu")
            A(f"s_addc_u32 {hi}, {hi}, 0", "salu")
        ops.append(advance)
    return ops


def rotate_ops(c: Config, st: Stream):
    """The ring moves on by one tile (scalar part), as closures for the slots of a step."""
    A = st.add
    return [
        lambda: A("s_mov_b32 %[tfill], %[cur]", "salu"),
        lambda: A("s_mov_b32 %[cur], %[tnext]", "salu"),
        lambda: A(f"s_add_u32 %[tnext], %[tnext], {c.stage}", "salu"),
        lambda: A("s_cmp_eq_u32 %[tnext], %[ringend]", "salu"),
        lambda: A("s_cselect_b32 %[tnext], %[lds0], %[tnext]", "salu"),
        lambda: A("s_add_u32 %[tm0], %[tfill], %[w1024]", "salu"),
        lambda: A("s_sub_i32 %[rem], %[rem], 1", "salu"),
        lambda: A("s_sub_i32 %[cnt], %[cnt], 1", "salu"),
    ]


def gen_ring_top(c: Config, st: Stream, tag: str):
    """Top of a tile iteration: wait for the tile ahead, barrier, rotate the ring, issue a new tile."""
    A = st.add
    if c.FL > 0:
        A("s_cmp_ge_i32 %[rem], 1", "salu")
        A(f"s_cbranch_scc1 .Lpart{tag}%=", "salu")
        A("s_waitcnt vmcnt(0)", "wait")
        A(f"s_branch .Lwaited{tag}%=", "salu")
        A(f".Lpart{tag}%=:", "label", nops=0)
        A(f"s_waitcnt vmcnt({c.FL * c.loads_min})", "wait")
        A(f".Lwaited{tag}%=:", "label", nops=0)
    else:
        A("s_waitcnt vmcnt(0)", "wait")
    if "barrier" not in c.ablate:
        A("s_barrier", "salu")
    # rotate: the stage of tile i-1 is refilled; cur = stage of tile i; next = stage of tile i+1
    A("s_mov_b32 %[tfill], %[cur]", "salu")
    A(f"s_add_u32 %[cur], %[cur], {c.stage}", "salu")
    A("s_cmp_eq_u32 %[cur], %[ringend]", "salu")
    A("s_cselect_b32 %[cur], %[lds0], %[cur]", "salu")
    A(f"s_add_u32 %[tnext], %[cur], {c.stage}", "salu")
    A("s_cmp_eq_u32 %[tnext], %[ringend]", "salu")
    A("s_cselect_b32 %[tnext], %[lds0], %[tnext]", "salu")
    A(f"s_cmp_gt_i32 %[rem], {c.FL}", "salu")
    if "noissue" in c.ablate:
        A(f"s_branch .Lnoissue{tag}%=", "salu")
    A(f"s_cbranch_scc0 .Lnoissue{tag}%=", "salu")
    # K slabs j * NW + wave, then V slabs; the last round only for the waves whose slab exists
    A("s_add_u32 %[tm0], %[tfill], %[w1024]", "salu")
    for kind, per, slabs, base, gbase, ptr in (("k", c.kper, c.kslabs, 0, c.GK, "kb"),
                                              ("v", c.vper, c.vslabs, c.kbytes, c.GV, "vb")):
        for j in range(per):
            partial = (j + 1) * c.NW > slabs
            if partial:
                A(f"s_cmp_lt_u32 %[wave], {slabs - j * c.NW}", "salu")
                A(f"s_cbranch_scc0 .Lskip{kind}{tag}%=", "salu")
            A(f"s_add_u32 m0, %[tm0], {base + j * c.NW * 1024}", "salu")
            A("s_nop 0", "nop")
            A(f"global_load_lds_dwordx4 {vr(gbase + j)}, s[{PTR_SGPR[ptr]}:{PTR_SGPR[ptr] + 1}]", "vmem", [gbase + j])
            if partial:
                A(f".Lskip{kind}{tag}%=:", "label", nops=0)
        lo, hi = f"s{PTR_SGPR[ptr]}", f"s{PTR_SGPR[ptr] + 1}"
        A(f"s_add_u32 {lo}, {lo}, %[{kind}step]", "salu")
        A(f"s_addc_u32 {hi}, {hi}, 0", "salu")
    A(f".Lnoissue{tag}%=:", "label", nops=0)
    A("s_sub_i32 %[rem], %[rem], 1", "salu")
    A(f"v_add_u32 {vr(c.KA)}, %[tnext], {vr(c.KLANE)}", "valu", [c.KLANE], [c.KA])
    A(f"v_add_u32 {vr(c.VA[0])}, %[cur], {vr(c.VLANE)}", "valu", [c.VLANE], [c.VA[0]])
    A(f"v_add_u32 {vr(c.VA[1])}, %[tnext], {vr(c.VLANE)}", "valu", [c.VLANE], [c.VA[1]])


def gen_fill(c: Config, st: Stream):
    """S(g) -> S[0], S(g+1) -> S[1], P(g) -> P[0] and the V operands of step g, for the first tile
    (stage `cur`).  Straight code with full waits: it runs once per statement."""
    A = st.add
    ka = c.PSUM  # address of the K rows of the tile at `cur`
    A(f"v_add_u32 {vr(ka)}, %[cur], {vr(c.KLANE)}", "valu", [c.KLANE], [ka])
    for kb in range(2):
        for t in range(c.NS):
            read_k(c, st, t, ka, kb)
        wait_lgkm(st, 0)
        for t in range(c.NS):
            mfma_qk(c, st, t, c.S[kb])
    A("s_nop 7", "nop", nops=8)
    A("s_nop 7", "nop", nops=8)
    for op in softmax_ops(c, st, c.S[0], c.P[0]):
        op()
    block_sum_check(c, st, 1, "fill")   # as after a step of parity 1: P[0] from S[0], newer scores in S[1]
    for t in range(c.NS):
        read_v(c, st, t, c.VA[0], 0)


def gen_drain(c: Config, st: Stream):
    """The last tile: O^T += V(g)^T P(g)^T with the softmax of S(g+1) under it, then step g+1."""
    NS = c.NS
    ops = softmax_ops(c, st, c.S[1], c.P[1])
    share = [len(ops) * (t + 1) // NS - len(ops) * t // NS for t in range(NS)]
    it = iter(ops)
    # S[1] may have come out of the matrix pipe right before (a statement of one tile)
    st.add("s_nop 7", "nop", nops=8)
    for t in range(NS):
        wait_lgkm(st, 2 * (NS - 1))       # V t+1 .. NS-1 of this step, V 0 .. t-1 of the next
        mfma_pv(c, st, t, c.P[0])
        read_v(c, st, t, c.VA[0], 1)
        for _ in range(share[t]):
            next(it)()
    # as after a step of parity 0: P[1] from S[1]; S[0] holds scores the row has already taken in, which no
    # reference needs to stay below
    block_sum_check(c, st, 0, "drain")
    st.add("s_nop 1", "nop", nops=2)
    for t in range(NS):
        wait_lgkm(st, 2 * (NS - 1 - t))
        mfma_pv(c, st, t, c.P[1])
    st.add("s_nop 7", "nop", nops=8)
    st.add("s_nop 7", "nop", nops=8)


def gen_issue_now(c: Config, st: Stream):
    for op in issue_ops(c, st):
        op()
    st.add("s_sub_i32 %[rem], %[rem], 1", "salu")


def gen_loop(c: Config):
    def S():
        return Stream()

    head, fill, fast, steps, top, drain, pre_drain = S(), S(), S(), S(), S(), S(), S()
    # operands that the compiler produced with vector instructions settle first
    head.add("s_nop 4", "nop", nops=5)
    head.add(f"s_add_u32 %[ringend], %[lds0], {c.NSTG * c.stage}", "salu")
    # The caller has waited, synchronised and rotated for the first tile (`cur` is its stage) but not
    # issued the tile that goes to the stage freed by that (`tfill`): that load is pending.
    head.add(f"s_add_u32 %[tnext], %[cur], {c.stage}", "salu")
    head.add("s_cmp_eq_u32 %[tnext], %[ringend]", "salu")
    head.add("s_cselect_b32 %[tnext], %[lds0], %[tnext]", "salu")
    head.add(f"s_sub_u32 %[tfill], %[cur], {c.stage}", "salu")
    head.add("s_cmp_eq_u32 %[cur], %[lds0]", "salu")
    head.add(f"s_cselect_b32 %[tfill], {(c.NSTG - 1) * c.stage}, %[tfill]", "salu")
    head.add("s_cselect_b32 %[tm0], %[lds0], 0", "salu")
    head.add("s_add_u32 %[tfill], %[tfill], %[tm0]", "salu")
    head.add("s_add_u32 %[tm0], %[tfill], %[w1024]", "salu")
    head.add(f"v_add_u32 {vr(c.KA)}, %[tnext], {vr(c.KLANE)}", "valu", [c.KLANE], [c.KA])
    head.add(f"v_add_u32 {vr(c.VA[0])}, %[cur], {vr(c.VLANE)}", "valu", [c.VLANE], [c.VA[0]])
    head.add(f"v_add_u32 {vr(c.VA[1])}, %[tnext], {vr(c.VLANE)}", "valu", [c.VLANE], [c.VA[1]])
    # EXEC of the loads of the last round: the lanes of the caller for the waves that have a slab in it, none
    # for the others; the statement leaves EXEC as it found it
    head.add("s_mov_b64 %[execsave], exec", "salu")
    head.add(f"s_cmp_lt_u32 %[wave], {c.kslabs - (c.kper - 1) * c.NW}", "salu")
    head.add("s_cselect_b64 %[klast], %[execsave], 0", "salu")
    head.add(f"s_cmp_lt_u32 %[wave], {c.vslabs - (c.vper - 1) * c.NW}", "salu")
    head.add("s_cselect_b64 %[vlast], %[execsave], 0", "salu")
    gen_fill(c, fill)
    # fast tile: the pending loads under step 0, the rotation under step 1 (the K address of the next
    # tile behind the last K read of step 1), then only the wait and the barrier between tiles
    gen_step(c, fast, 0, filler=issue_ops(c, fast), tag="fast")
    gen_step(c, fast, 1, filler=rotate_ops(c, fast), tag="fast",
             late_filler=[lambda: fast.add(f"v_add_u32 {vr(c.KA)}, %[tnext], {vr(c.KLANE)}", "valu", [c.KLANE], [c.KA])])
    fast.add(f"s_waitcnt vmcnt({c.FL * c.loads_min})", "wait")
    if "barrier" not in c.ablate:
        fast.add("s_barrier", "salu")
    fast.add(f"v_mov_b32 {vr(c.VA[0])}, {vr(c.VA[1])}", "valu", [c.VA[1]], [c.VA[0]])
    fast.add(f"v_add_u32 {vr(c.VA[1])}, %[tnext], {vr(c.VLANE)}", "valu", [c.VLANE], [c.VA[1]])
    gen_step(c, steps, 0, tag="rest")
    gen_step(c, steps, 1, tag="rest")
    gen_ring_top(c, top, "")
    gen_issue_now(c, pre_drain)
    gen_drain(c, drain)
    # what can follow what, with no reference raised and with every one of them raised
    def raised(ins):
        out = []
        for i in ins:
            out.append(i)
            if i["kind"] == "raise":
                body = S()
                gen_raise(c, body, i["par"])
                out += body.ins
        return out

    if not c.ablate:
        for how, path in (("", lambda x: x), (", references raised", raised)):
            check_stream(path(head.ins + fill.ins + pre_drain.ins + drain.ins), c.name + " (one tile)" + how)
            check_stream(path(head.ins + fill.ins + fast.ins + fast.ins + fast.ins + pre_drain.ins + drain.ins),
                         c.name + " (fast)" + how)
            check_stream(path(head.ins + fill.ins + fast.ins + fast.ins + steps.ins + top.ins + steps.ins + top.ins + drain.ins),
                         c.name + " (fast, then the last tiles)" + how)
    out = S()
    out.ins += head.ins + fill.ins
    # fast tiles while a load is pending and a tile follows
    out.add(".Lfast%=:", "label", nops=0)
    out.add("s_cmp_le_i32 %[cnt], 1", "salu")
    out.add("s_cbranch_scc1 .Lpredrain%=", "salu")
    out.add(f"s_cmp_le_i32 %[rem], {c.FL}", "salu")
    out.add("s_cbranch_scc1 .Lrest%=", "salu")
    out.ins += fast.ins
    out.add("s_branch .Lfast%=", "salu")
    # the last tile of the statement is next: the pending load, if there is one
    out.add(".Lpredrain%=:", "label", nops=0)
    out.add(f"s_cmp_le_i32 %[rem], {c.FL}", "salu")
    out.add("s_cbranch_scc1 .Ldrain%=", "salu")
    out.ins += pre_drain.ins
    out.add("s_branch .Ldrain%=", "salu")
    # nothing left to load: plain steps, then the wait, the barrier and the rotation
    out.add(".Lrest%=:", "label", nops=0)
    out.add("s_cmp_le_i32 %[cnt], 1", "salu")
    out.add("s_cbranch_scc1 .Ldrain%=", "salu")
    out.ins += steps.ins
    out.add("s_sub_i32 %[cnt], %[cnt], 1", "salu")
    out.ins += top.ins
    out.add("s_branch .Lrest%=", "salu")
    out.add(".Ldrain%=:", "label", nops=0)
    out.ins += drain.ins
    # out of line: the blocks that raise the reference of the rows, one per place that may ask for it
    places = [i for i in out.ins if i["kind"] == "raise"]
    if places:
        out.add("s_branch .Lend%=", "salu")
        for i in places:
            out.add(f".Lraise{i['tag']}%=:", "label", nops=0)
            gen_raise(c, out, i["par"])
            out.add(f"s_branch .Lback{i['tag']}%=", "salu")
        out.add(".Lend%=:", "label", nops=0)
    return out.ins


# scalar temporaries of the statement, and the special registers it writes (EXEC is saved and restored)
TEMP_SGPRS = ("tfill", "tnext", "tm0", "ringend", "klast", "vlast", "execsave")
SPECIAL_CLOBBERS = ["vcc", "scc", "m0"]


def operand_lists(c: Config):
    outs, ins, clob = [], [], []
    for db in range(c.DB):
        outs.append((f"o{db}", f"+{{v[{c.O + 16 * db}:{c.O + 16 * db + 15}]}}"))
    outs.append(("l", f"+{{v{c.L}}}"))
    for n in ("cnt", "rem", "cur"):
        outs.append((n, "+s"))
    for n in ("kb", "vb"):
        outs.append((n, f"+{{s[{PTR_SGPR[n]}:{PTR_SGPR[n] + 1}]}}"))
    outs.append(("mneg", f"+{{v[{c.MNEG}:{c.MNEG + 15}]}}"))
    for n in TEMP_SGPRS:
        outs.append((n, "=&s"))
    nq = 4 * c.NS
    for i in range(0, nq, 16):
        w = min(16, nq - i)
        ins.append((f"q{i // 16}", f"{{v[{c.Q + i}:{c.Q + i + w - 1}]}}"))
    ins.append(("klane", f"{{v{c.KLANE}}}"))
    ins.append(("vlane", f"{{v{c.VLANE}}}"))
    for j in range(c.kper):
        ins.append((f"gk{j}", f"{{v{c.GK + j}}}"))
    for j in range(c.vper):
        ins.append((f"gv{j}", f"{{v{c.GV + j}}}"))
    for n in ("lds0", "kstep", "vstep", "w1024", "wave"):
        ins.append((n, "s"))
    if c.elem == "f16":
        ins.append(("blockhi", "s"))
    used = set(rng(c.O, 16 * c.DB)) | {c.L} | set(rng(c.Q, nq)) | set(rng(c.MNEG, 16)) | {c.KLANE, c.VLANE}
    used |= set(rng(c.GK, c.kper)) | set(rng(c.GV, c.vper))
    for r in range(c.nvgpr):
        if r not in used:
            clob.append(f"v{r}")
    return outs, ins, clob


def emit_macro(c: Config, out):
    ins = gen_loop(c)
    outs, inputs, clob = operand_lists(c)
    check_clobbers(ins, outs, clob + SPECIAL_CLOBBERS, c.name)
    temps = TEMP_SGPRS
    names = [n for n, _ in outs if n not in temps] + [n for n, _ in inputs]
    out.write(f"// {c.name}: {c.elem} D={c.D}, {c.NW} waves, {c.NSTG} stages; {c.nvgpr} vector registers\n")
    out.write(f"#define {c.name}_VGPRS {c.nvgpr}\n")
    out.write(f"#define {c.name}({', '.join('A_' + n for n in names)}) \\\n")
    out.write("    do { unsigned t_fill_, t_next_, t_m0_, t_end_; unsigned long long t_kl_, t_vl_, t_ex_; asm volatile( \\\n")
    for i in ins:
        out.write(f'        "{i["text"]}\\n\\t" \\\n')
    tmpmap = {"tfill": "t_fill_", "tnext": "t_next_", "tm0": "t_m0_", "ringend": "t_end_", "klast": "t_kl_", "vlast": "t_vl_",
              "execsave": "t_ex_"}
    o_s = ", ".join(f'[{n}] "{cs}"({tmpmap.get(n, "A_" + n)})' for n, cs in outs)
    i_s = ", ".join(f'[{n}] "{cs}"(A_{n})' for n, cs in inputs)
    c_s = ", ".join(f'"{x}"' for x in ["memory"] + SPECIAL_CLOBBERS + clob)
    out.write(f"        : {o_s} \\\n        : {i_s} \\\n        : {c_s}); }} while (0)\n\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("-o", "--output", default="chill_fwd_loop.inc")
    ap.add_argument("--ablate", default="", help="timing experiments: comma-separated parts to leave out "
                                                 "(barrier, valu, mfma); the results are wrong")
    args = ap.parse_args()
    ab = [x for x in args.ablate.split(",") if x]
    global ABLATE_WAITS
    ABLATE_WAITS = any(x in ab for x in ("lds", "kread", "vread", "vb128"))
    configs = [Config("bf16", 128, 8, 4, ab), Config("f16", 128, 8, 4, ab),
               Config("bf16", 64, 4, 3, ab), Config("f16", 64, 4, 3, ab)]
    with open(args.output, "w") as out:
        out.write("// Generated by gen_fwd_loop.py; do not edit.\n#pragma once\n\n")
        for c in configs:
            emit_macro(c, out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
