#!/usr/bin/env python3
"""Generates the hand-scheduled inner loop of the dK/dV kernel with register-resident K
(chill_bwd_dkdv_regs.h, two 32-key blocks per wave) as an inline-asm statement: chill_bwd_loop.inc,
one macro per element type.

One wave of a 4-wave workgroup (one wave per SIMD) owns 64 key rows: K as MFMA B operands in
registers, its dK^T / dV^T accumulators (2 x 2 x D/32 blocks) in the accumulation registers, V in LDS.
An ITERATION takes one 32-row tile of Q and dO, with the LSE2 and delta of its rows, from a ring of
four LDS stages and runs 64 MFMAs (D = 128), reference chill_attention/chill_bwd_dkdv.py:362-403:

    phase A  slots  0..15   S_c    = Q K_c^T                 (c = 0, 1: the wave's two key blocks; S_0 first, so that
                                                          its exponentials can start eight slots earlier)
    phase B  slots 16..31   dP'_c  = delta - dO V_c^T        (V is stored negated; the chain starts from delta)
    phase C  slots 32..47   dV_c^T += dO^T P_c               P = exp2(S * scale - LSE2)
    phase D  slots 48..63   dK'_c^T += Q^T dS'_c             dS' = P * dP' = -dS   (the caller scales by -sm_scale)

Every streamed operand read from LDS feeds two MFMAs (one per key block).  The vector work rides in
the slots: the exponentials in those of phase B and the first half of phase C, the products behind
them.  Operands are read into a ring of register units as early as units are free; every
`s_waitcnt lgkmcnt` is computed from the order of the reads.  At the end of an iteration the first
operands of the next one (its LSE2, delta and Q chunks) are already on their way.

The statement runs `cnt` consecutive iterations of one wave, each: issue the tile three ahead into the stage
that has just been freed, 64 slots; the wait for the tile ahead and the barrier of the next iteration stand in
front of slot 56, where every read of the current tile has returned, so that the last MFMAs cover the barrier.

Measured on the causal bf16 B8 H16 T8192 workload (timing builds with parts of the loop left out, --ablate):
the kernel takes 3.55 ms; without the LDS reads of the loop 3.15, without its vector instructions 3.35, without
both 3.04, without its MFMAs 2.13, with none of the three (barriers, waits and everything outside the loop remain)
0.85 ms.  A lone wave per SIMD issues at most one instruction every four cycles: ~330 instructions per 64 MFMAs
leave little room, so the generator spreads the vector work over as many slots as the data dependences allow.  The caller guarantees that every
tile of the run is predicate-free for the wave, that the tiles it issues exist in full and belong to one
query head (the pointers advance by a fixed step), and does everything else itself.
"""
from __future__ import annotations

import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from asm_stream import AGPR, LGKM_MAX, Sched, Stream, areg, check_clobbers, check_stream, deal, rng, vr  # noqa: E402,F401

# fixed scalar register pairs of the four tile pointers (their halves are added to separately)
PTR_SGPR = {"q": 88, "do": 90, "lse": 92, "del": 94}
ABLATE = set()  # timing experiments only (--ablate): parts of the loop left out; the results are wrong
TEMP_SGPRS = ("execsave",)
SPECIAL_CLOBBERS = ["vcc", "scc", "m0"]


class Config:
    # Slot windows of the vector work, per head dim: exponentials of block 0, of the two halves of block 1
    # (split_a) or of everything (not split_a), products and packs of entries 0..7 and 8..15, the slot the
    # next iteration's barrier stands in front of, the last slot that carries tile loads.
    WINDOWS = {
        128: dict(e0=(10, 23), e1a=(24, 31), e1b=(32, 39), e=(18, 39), g0=(40, 45), p0=(44, 47), g1=(46, 51),
                  p1=(52, 55), barrier=56, dma=15),
        64: dict(e0=(6, 11), e1a=(12, 15), e1b=(16, 19), e=(9, 19), g0=(20, 22), p0=(22, 23), g1=(23, 25),
                 p1=(26, 27), barrier=28, dma=7),
    }

    def __init__(self, elem: str, D: int = 128, units: int = 10, barrier_slot: int = None, split_a: bool = True):
        assert elem in ("bf16", "f16") and D in self.WINDOWS
        self.win = self.WINDOWS[D]
        if barrier_slot is None:
            barrier_slot = self.win["barrier"]
        self.elem, self.D = elem, D
        self.CB, self.NSTG, self.NW = 2, 4, 4
        self.NJ = D // 16                 # MFMAs of a 32 x 32 product over the head dim
        self.DB = D // 32
        self.row_bytes = 2 * D
        self.tile = 32 * self.row_bytes   # a 32-row tile, also a 32-row block of the V tile
        self.vec = 32 * 4
        self.stage = 2 * self.tile + 2 * self.vec
        self.units = units
        r = 0
        self.S = (r, r + 16); r += 32
        self.DP = (r, r + 16); r += 32
        self.LSE = r; r += 16
        self.PB = (r, r + 8); r += 16
        self.RING = r; r += 4 * units
        self.T = r; r += 4
        self.nvgpr = r
        self.slots = 8 * self.NJ          # 64
        self.split_a = split_a
        self.barrier_slot = barrier_slot  # the barrier of the next iteration stands in front of this slot's MFMA
        self.mfma = "v_mfma_f32_32x32x16_" + elem
        self.cvt = "v_cvt_pk_bf16_f32" if elem == "bf16" else "v_cvt_pk_f16_f32"
        self.name = f"CHILL_DKDV_LOOP_{elem.upper()}_{D}"
        # rows 16 apart share the swizzle key of their chunks only in rows of 256 bytes and more: below that the
        # transposed operands of the two 16-row halves of a tile have per-lane addresses of their own
        self.half_affine = self.row_bytes >= 256
        self.slabs = self.tile // (self.NW * 1024)   # 1 KiB slabs of a tile that one wave loads: 2, or 1 at head dim 64
        self.loads_per_tile = 2 * self.slabs         # per wave: Q and dO (the wave with the vectors: two more)

    def dv(self, c, db):
        return AGPR + 16 * (c * self.DB + db)

    def dk(self, c, db):
        return AGPR + 16 * (self.CB * self.DB + c * self.DB + db)


class AblatingStream(Stream):
    """Drops the MFMAs of a timing experiment."""

    def add(self, text, kind, *a, **kw):
        if kind == "mfma" and "mfma" in ABLATE:
            return
        super().add(text, kind, *a, **kw)


def softmax_pairs(c: Config, st: Stream, blk: int, pairs):
    """P = exp2(S * scale - LSE2) for entry pairs `pairs` of key block `blk`, packed into PB: closures of
    one instruction each, the pack of a pair behind the exponentials of the next."""
    ops = []
    S, PB = c.S[blk], c.PB[blk]
    pend = None
    for k in pairs:
        t0, t1 = c.T + (2 * k) % 4, c.T + (2 * k + 1) % 4
        for e, t in ((2 * k, t0), (2 * k + 1, t1)):
            ops.append(lambda e=e, t=t: st.add(f"v_fma_f32 {vr(t)}, {vr(S + e)}, %[scale], -{vr(c.LSE + e)}", "valu",
                                               [S + e, c.LSE + e], [t]))
        for e, t in ((2 * k, t0), (2 * k + 1, t1)):
            ops.append(lambda e=e, t=t: st.add(f"v_exp_f32 {vr(S + e)}, {vr(t)}", "trans", [t], [S + e]))
        if pend is not None:
            ops.append(pend)
        pend = (lambda k=k: st.add(f"{c.cvt} {vr(PB + k)}, {vr(S + 2 * k)}, {vr(S + 2 * k + 1)}", "valu",
                                   [S + 2 * k, S + 2 * k + 1], [PB + k]))
    ops.append(pend)
    return ops


def product_ops(c: Config, st: Stream, blk: int, entries):
    S, DP = c.S[blk], c.DP[blk]
    return [(lambda e=e: st.add(f"v_mul_f32 {vr(DP + e)}, {vr(S + e)}, {vr(DP + e)}", "valu", [S + e, DP + e], [DP + e]))
            for e in entries]


def pack_ops(c: Config, st: Stream, blk: int, pairs):
    DP, PB = c.DP[blk], c.PB[blk]
    return [(lambda k=k: st.add(f"{c.cvt} {vr(PB + k)}, {vr(DP + 2 * k)}, {vr(DP + 2 * k + 1)}", "valu",
                                [DP + 2 * k, DP + 2 * k + 1], [PB + k])) for k in pairs]


def dma_ops(c: Config, st: Stream, tgt: int):
    """The loads of the tile three ahead into stage `tgt`, and the pointers moved on by one tile."""
    A = st.add
    ops = []
    base = tgt * c.stage
    for name, off in (("q", 0), ("do", c.tile)):
        for i in range(c.slabs):
            def load(name=name, off=off, i=i):
                A(f"s_add_u32 m0, %[dmabase], {base + off + i * c.NW * 1024}", "salu")
                A("s_nop 0", "nop")
                A(f"global_load_lds_dwordx4 %[g{name}{i}], s[{PTR_SGPR[name]}:{PTR_SGPR[name] + 1}]", "vmem")
            ops.append(load)

    def vectors():
        # LSE2 and delta of the tile's 32 rows: the lower half of one wave
        A("s_cmp_eq_u32 %[vecwave], 0", "salu")
        A(f"s_cbranch_scc1 .Lnovec{tgt}%=", "salu")
        A("s_mov_b64 exec, 0xffffffff", "salu")
        for name, off in (("lse", 0), ("del", c.vec)):
            A(f"s_add_u32 m0, %[vecdma], {base + off}", "salu")
            A("s_nop 0", "nop")
            A(f"global_load_lds_dword %[lane4], s[{PTR_SGPR[name]}:{PTR_SGPR[name] + 1}]", "vmem")
        A("s_mov_b64 exec, %[execsave]", "salu")
        A(f".Lnovec{tgt}%=:", "label", nops=0)
    ops.append(vectors)
    for name, step in (("q", "%[qstep]"), ("do", "%[dostep]"), ("lse", str(c.vec)), ("del", str(c.vec))):
        lo, hi = f"s{PTR_SGPR[name]}", f"s{PTR_SGPR[name] + 1}"

        def advance(lo=lo, hi=hi, step=step):
            A(f"s_add_u32 {lo}, {lo}, {step}", "salu")
            A(f"s_addc_u32 {hi}, {hi}, 0", "salu")
        ops.append(advance)
    return ops


class Iteration:
    """One iteration (stage `s`), from the instruction after the barrier to the last MFMA."""

    def __init__(self, c: Config, q_units):
        self.c = c
        self.q_units = list(q_units)      # ring unit that holds Q chunk j when the iteration starts

    def prefetch_reads(self, c, s, q_units):
        """(key, text, registers) of what an iteration expects to be on its way when it starts, for
        the tile in stage s, in the canonical order."""
        out = []
        for g in range(4):
            out.append((("lse", g), f"ds_read_b128 {vr(c.LSE + 4 * g, 4)}, %[vec] offset:{s * c.stage + 32 * g}",
                        rng(c.LSE + 4 * g, 4)))
        for j in range(c.NJ):
            u = c.RING + 4 * q_units[j]
            out.append((("q", j), f"ds_read_b128 {vr(u, 4)}, %[qrow{j}] offset:{s * c.stage}", rng(u, 4)))
        for blk in range(c.CB):
            for g in range(4):
                out.append((("del", blk, g), f"ds_read_b128 {vr(c.DP[blk] + 4 * g, 4)}, %[vec] offset:{s * c.stage + c.vec + 32 * g}",
                            rng(c.DP[blk] + 4 * g, 4)))
        return out

    def generate(self, st: Stream, s: int, with_dma=True, with_prefetch=True, with_barrier=True):
        """Returns the ring units that hold the Q chunks of the next iteration.  Without `with_dma` this is an
        iteration of a run's tail: it requests no tile, and its barrier waits for every tile still on its way."""
        c = self.c
        self.tail = not with_dma
        nxt, tgt = (s + 1) % c.NSTG, (s + 3) % c.NSTG
        NS = c.slots
        carried = [regs for _, _, regs in self.prefetch_reads(c, s, self.q_units)]
        # the canonical order of the prefetch is the order the steady state issues it in (see below)
        carried = self.carried_order(carried)
        sch = Sched(st, carried)
        unit_of = {("q", j): self.q_units[j] for j in range(c.NJ)}
        free = [u for u in range(c.units) if u not in self.q_units]
        release_at = {}   # slot -> units freed by the MFMA of that slot

        def consumer(key, slot):
            release_at.setdefault(slot, []).append(key)

        # ---- the MFMAs, slot by slot: (text pieces, operand keys)
        slots = []
        if c.split_a:
            # S_0 in full, then S_1: the exponentials of block 0 can start eight slots earlier (a Q chunk stays in
            # its ring unit for both)
            for blk in range(c.CB):
                for j in range(c.NJ):
                    slots.append(("A", j, blk))
        else:
            for j in range(c.NJ):
                for blk in range(c.CB):
                    slots.append(("A", j, blk))
        for j in range(c.NJ):
            for blk in range(c.CB):
                slots.append(("B", j, blk))
        for sx in range(2):
            for db in range(c.DB):
                for blk in range(c.CB):
                    slots.append(("C", sx, db, blk))
        for sx in range(2):
            for db in range(c.DB):
                for blk in range(c.CB):
                    slots.append(("D", sx, db, blk))
        assert len(slots) == NS
        # last consumer of every ring operand
        last_use = {}
        for t, sl in enumerate(slots):
            if sl[0] == "A":
                last_use[("q", sl[1])] = t
            elif sl[0] == "B":
                last_use[("do", sl[1])] = t
                last_use[("v", sl[2], sl[1])] = t
            elif sl[0] == "C":
                last_use[("dot", sl[1], sl[2])] = t
            else:
                last_use[("qt", sl[1], sl[2])] = t

        # ---- the queue of reads of this iteration, in the order of their use, then the prefetch
        queue = []   # (key, ready_slot, kind)
        for j in range(c.NJ):
            queue.append((("do", j), 0))
            for blk in range(c.CB):
                queue.append((("v", blk, j), 0))
        for sx in range(2):
            for db in range(c.DB):
                queue.append((("dot", sx, db), 0))
        for sx in range(2):
            for db in range(c.DB):
                queue.append((("qt", sx, db), 0))
        w = c.win
        E_LO, E_HI = w["e"]          # slots of the exponentials
        G0_LO, G0_HI = w["g0"]       # products of entries 0..7
        P0_LO, P0_HI = w["p0"]       # their pack (PB[0:3] is free once the dV^T MFMAs of the first half have been issued)
        G1_LO, G1_HI = w["g1"]
        P1_LO, P1_HI = w["p1"]
        if with_prefetch:
            for g in range(4):
                queue.append((("nlse", g), E_HI + 1))
            for j in range(c.NJ):
                queue.append((("nq", j), 0))
            for blk in range(c.CB):
                for g in range(4):
                    # (dP' is last read when dS' is packed)
                    queue.append((("ndel", blk, g), P1_HI + 1))

        def read_text(key, unit):
            u = c.RING + 4 * unit if unit is not None else None
            kind = key[0]
            if kind == "do":
                return [(f"ds_read_b128 {vr(u, 4)}, %[qrow{key[1]}] offset:{s * c.stage + c.tile}", rng(u, 4))]
            if kind == "v":
                return [(f"ds_read_b128 {vr(u, 4)}, %[vrow{key[2]}] offset:{key[1] * c.tile}", rng(u, 4))]
            if kind in ("dot", "qt"):
                off = s * c.stage + (c.tile if kind == "dot" else 0) + (key[1] * 16 * c.row_bytes if c.half_affine else 0)
                at = f"qtr{key[2]}" if c.half_affine else f"qtr{key[2]}_{key[1]}"
                return [(f"ds_read_b64_tr_b16 {vr(u, 2)}, %[{at}_0] offset:{off}", rng(u, 2)),
                        (f"ds_read_b64_tr_b16 {vr(u + 2, 2)}, %[{at}_1] offset:{off}", rng(u + 2, 2))]
            if kind == "nq":
                return [(f"ds_read_b128 {vr(u, 4)}, %[qrow{key[1]}] offset:{nxt * c.stage}", rng(u, 4))]
            if kind == "nlse":
                g = key[1]
                return [(f"ds_read_b128 {vr(c.LSE + 4 * g, 4)}, %[vec] offset:{nxt * c.stage + 32 * g}", rng(c.LSE + 4 * g, 4))]
            if kind == "ndel":
                blk, g = key[1], key[2]
                return [(f"ds_read_b128 {vr(c.DP[blk] + 4 * g, 4)}, %[vec] offset:{nxt * c.stage + c.vec + 32 * g}",
                         rng(c.DP[blk] + 4 * g, 4))]
            raise KeyError(key)

        # ---- vector work by slot
        valu = [[] for _ in range(NS)]

        def place(ops, lo, hi):
            if "valu" in ABLATE:
                return
            for t, lst in enumerate(deal(ops, lo, hi, NS)):
                valu[t] += lst
        if c.split_a:
            place(softmax_pairs(c, st, 0, range(0, 8)), *w["e0"])
            place(softmax_pairs(c, st, 1, range(0, 4)), *w["e1a"])
            place(softmax_pairs(c, st, 1, range(4, 8)), *w["e1b"])
        else:
            e_ops = []
            for half in (range(0, 4), range(4, 8)):
                for blk in range(c.CB):
                    e_ops += softmax_pairs(c, st, blk, half)
            place(e_ops, E_LO, E_HI)
        place(product_ops(c, st, 0, range(0, 8)) + product_ops(c, st, 1, range(0, 8)), G0_LO, G0_HI)
        place(pack_ops(c, st, 0, range(0, 4)) + pack_ops(c, st, 1, range(0, 4)), P0_LO, P0_HI)
        place(product_ops(c, st, 0, range(8, 16)) + product_ops(c, st, 1, range(8, 16)), G1_LO, G1_HI)
        place(pack_ops(c, st, 0, range(4, 8)) + pack_ops(c, st, 1, range(4, 8)), P1_LO, P1_HI)
        if with_dma and "dma" not in ABLATE:
            scalar = deal(dma_ops(c, st, tgt), 0, w["dma"], NS)
        elif "dma" not in ABLATE:
            # (the vector instructions behind the score MFMAs count on the issue slots the tile loads take)
            pads = []
            for op in dma_ops(c, count := Stream(), tgt):
                before = len(count.ins)
                op()
                n_ins = len(count.ins) - before
                pads.append(lambda n_ins=n_ins: st.add(f"s_nop {n_ins - 1}", "nop", nops=n_ins))
            scalar = deal(pads, 0, w["dma"], NS)
        else:
            scalar = [[] for _ in range(NS)]

        next_q = {}
        READS_PER_SLOT = 3
        self.prefetch_order = []
        last_tile_read = 0   # sequence number of the last read of this iteration's tile
        for t, sl in enumerate(slots):
            if t == c.barrier_slot and with_barrier:
                self.early_barrier(st, sch, s, queue, last_tile_read)
            # operands and the MFMA
            if sl[0] == "A":
                _, j, blk = sl
                a = c.RING + 4 * unit_of[("q", j)]
                sch.need(rng(a, 4))
                cin = "0" if j == 0 else vr(c.S[blk], 16)
                st.add(f"{c.mfma} {vr(c.S[blk], 16)}, {vr(a, 4)}, %[k{blk}_{j}], {cin}", "mfma",
                       rng(a, 4) + ([] if j == 0 else rng(c.S[blk], 16)), rng(c.S[blk], 16))
            elif sl[0] == "B":
                _, j, blk = sl
                a = c.RING + 4 * unit_of[("do", j)]
                b = c.RING + 4 * unit_of[("v", blk, j)]
                sch.need(rng(a, 4) + rng(b, 4) + (rng(c.DP[blk], 16) if j == 0 else []))
                st.add(f"{c.mfma} {vr(c.DP[blk], 16)}, {vr(a, 4)}, {vr(b, 4)}, {vr(c.DP[blk], 16)}", "mfma",
                       rng(a, 4) + rng(b, 4) + rng(c.DP[blk], 16), rng(c.DP[blk], 16))
            else:
                ph, sx, db, blk = sl
                a = c.RING + 4 * unit_of[("dot" if ph == "C" else "qt", sx, db)]
                acc = c.dv(blk, db) if ph == "C" else c.dk(blk, db)
                b = c.PB[blk] + 4 * sx
                sch.need(rng(a, 4))
                st.add(f"{c.mfma} {areg(acc, 16)}, {vr(a, 4)}, {vr(b, 4)}, {areg(acc, 16)}", "mfma",
                       rng(a, 4) + rng(b, 4) + rng(acc, 16), rng(acc, 16))
            # units whose last consumer this was
            for key, last in last_use.items():
                if last == t:
                    free.append(unit_of.pop(key))
            # reads
            issued = 0
            while queue and issued < READS_PER_SLOT:
                key, ready = queue[0]
                if ready > t:
                    break
                needs_unit = key[0] in ("do", "v", "dot", "qt", "nq")
                if needs_unit and not free:
                    break
                unit = free.pop(free.index(min(free))) if needs_unit else None
                for text, regs in read_text(key, unit):
                    if "lds" not in ABLATE:
                        sch.read(text, None, regs)
                if key[0] in ("do", "dot", "qt"):
                    last_tile_read = sch.seq
                if key[0] == "nq":
                    next_q[key[1]] = unit
                elif needs_unit:
                    unit_of[key] = unit
                if key[0] in ("nq", "nlse", "ndel"):
                    self.prefetch_order.append(key)
                queue.pop(0)
                issued += 1
            # vector and scalar work of the slot
            for op in valu[t]:
                # (an operand that an LDS read delivers, LSE2, is waited for first)
                op()
                ins = st.ins[-1]
                pend = [r for r in ins["reads"] | ins["writes"] if r in sch.pending]
                if pend:
                    st.ins.pop()
                    sch.need(pend)
                    op()
            for op in scalar[t]:
                op()
        if c.barrier_slot >= NS and with_barrier:
            self.early_barrier(st, sch, s, queue, last_tile_read)
        assert not queue, f"reads left over: {queue}"
        self.pending_after = dict(sch.pending)
        return [next_q[j] for j in range(c.NJ)] if with_prefetch else None

    def carried_order(self, carried):
        return carried

    def early_barrier(self, st, sch, s, queue, last_tile_read):
        """The barrier of the NEXT iteration, early enough for the MFMAs behind it to cover its latency: every
        read of this iteration's tile has returned (the stage is refilled after the barrier), and the tile two
        ahead has landed.  The last iteration of a run leaves that barrier to the caller."""
        c = self.c
        assert not any(k[0] in ("do", "dot", "qt") for k, _ in queue), "reads of the tile behind the barrier"
        sch.wait_upto(last_tile_read)
        sfx = f"t{s}" if self.tail else f"{s}"
        st.add("s_cmp_eq_u32 %[cnt], 1", "salu")
        st.add(f"s_cbranch_scc1 .Lnobar{sfx}%=", "salu")
        st.add(f"s_waitcnt vmcnt({0 if self.tail else c.loads_per_tile})", "wait")
        if "barrier" not in ABLATE:
            st.add("s_barrier", "salu")
        st.add(f".Lnobar{sfx}%=:", "label", nops=0)


def find_steady_state(c: Config):
    """The ring units that hold the prefetched Q chunks at the start of an iteration, per stage: a cycle
    of assignments whose length divides the number of stages (the iteration of stage s starts from
    cycle[s % len] and leaves cycle[(s + 1) % len] behind), with the order in which each issues its prefetch."""
    states = [list(range(c.NJ))]
    orders = []
    for _ in range(64):
        it = Iteration(c, states[-1])
        nq = it.generate(Stream(), 0)
        orders.append(it.prefetch_order)
        if nq in states:
            first = states.index(nq)
            if c.NSTG % (len(states) - first) == 0:
                return states[first:], orders[first:]
            raise SystemExit(f"{c.name}: the ring settles into a cycle of {len(states) - first} iterations")
        states.append(nq)
    raise SystemExit(f"{c.name}: the ring does not settle into a steady state")


class SteadyIteration(Iteration):
    """An iteration whose carried reads are in the order the steady state issues its prefetch in."""

    def __init__(self, c, q_units, order):
        super().__init__(c, q_units)
        self.order = order

    def reads_for_stage(self, s):
        c = self.c
        by_key = {}
        for key, text, regs in self.prefetch_reads(c, s, self.q_units):
            by_key[key] = (text, regs)
        out = []
        for key in self.order:
            k = {"nlse": ("lse", key[1]), "nq": ("q", key[1]), "ndel": ("del",) + tuple(key[1:])}[key[0]]
            out.append(by_key[k])
        return out

    def generate(self, st, s, **kw):
        self._stage = s
        return super().generate(st, s, **kw)

    def carried_order(self, carried):
        return [regs for _, regs in self.reads_for_stage(self._stage)]


def gen_statement(c: Config):
    cycle, orders = find_steady_state(c)
    n = len(cycle)
    # the iteration of stage s, and the one that prefetches for it (whose order its carried reads are in)
    its = [SteadyIteration(c, cycle[s % n], orders[(s - 1) % n]) for s in range(c.NSTG)]
    out = Stream()
    A = out.add
    A("s_mov_b64 %[execsave], exec", "salu")
    for s in range(1, c.NSTG):
        A(f"s_cmp_eq_u32 %[st0], {s}", "salu")
        A(f"s_cbranch_scc1 .Lpro{s}%=", "salu")
    bodies, pros, tails = [], [], []
    for s in range(c.NSTG):
        pro = Stream()
        pro.add(f".Lpro{s}%=:", "label", nops=0)
        # (the caller may have written to LDS just before: V negated in place, rows past the end of a tile zeroed)
        pro.add(f"s_waitcnt vmcnt({c.loads_per_tile}) lgkmcnt(0)", "wait", wait=0)
        pro.add("s_barrier", "salu")
        sch = Sched(pro)
        for text, regs in its[s].reads_for_stage(s):
            sch.read(text, None, regs)
        # a run that starts inside its tail (at most `tailn` iterations, none of which requests a tile)
        pro.add("s_cmp_le_u32 %[cnt], %[tailn]", "salu")
        pro.add(f"s_cbranch_scc1 .Ltbody{s}%=", "salu")
        pro.add(f"s_branch .Lbody{s}%=", "salu")
        pros.append(pro)
        body = AblatingStream()
        body.add(f".Lbody{s}%=:", "label", nops=0)
        nq = its[s].generate(body, s)
        assert nq == cycle[(s + 1) % n] and its[s].prefetch_order == orders[s % n]
        body.add("s_sub_u32 %[cnt], %[cnt], 1", "salu")
        body.add("s_cmp_le_u32 %[cnt], %[tailn]", "salu")
        body.add(f"s_cbranch_scc1 .Ltsel{(s + 1) % c.NSTG}%=", "salu")
        if s == c.NSTG - 1:
            body.add("s_branch .Lbody0%=", "salu")
        bodies.append(body)
        # the same iteration for the last `tailn` tiles of a run that ends with the workgroup's last tile: the
        # tiles three ahead do not exist
        tb = AblatingStream()
        tb.add(f".Ltsel{s}%=:", "label", nops=0)
        tb.add("s_cmp_eq_u32 %[cnt], 0", "salu")
        tb.add("s_cbranch_scc1 .Lexit%=", "salu")
        tb.add(f".Ltbody{s}%=:", "label", nops=0)
        nq = its[s].generate(tb, s, with_dma=False)
        assert nq == cycle[(s + 1) % n] and its[s].prefetch_order == orders[s % n]
        tb.add("s_sub_u32 %[cnt], %[cnt], 1", "salu")
        if s == c.NSTG - 1:
            tb.add("s_branch .Ltsel0%=", "salu")
        tails.append(tb)
    tail = Stream()
    tail.add(".Lexit%=:", "label", nops=0)
    tail.add("s_waitcnt lgkmcnt(0)", "wait", wait=0)
    # the hazards of every path: a prologue, its body, the next body, the exit; the same through the tail
    for s in range(c.NSTG if not ABLATE else 0):
        n1, n2 = (s + 1) % c.NSTG, (s + 2) % c.NSTG
        for name, path in (("from stage", pros[s].ins + bodies[s].ins + bodies[n1].ins + bodies[n2].ins + tail.ins),
                           ("one iteration, stage", pros[s].ins + bodies[s].ins + tail.ins),
                           ("into the tail, stage", pros[s].ins + bodies[s].ins + tails[n1].ins + tails[n2].ins + tail.ins),
                           ("tail only, stage", pros[s].ins + tails[s].ins + tails[n1].ins + tail.ins),
                           ("one tail iteration, stage", pros[s].ins + tails[s].ins + tail.ins)):
            check_stream(path, f"{c.name} ({name} {s})")
    # the first prologue follows the dispatch directly
    out.ins += pros[0].ins
    for s in range(c.NSTG):
        out.ins += bodies[s].ins
    for s in range(c.NSTG):
        out.ins += tails[s].ins
    for s in range(1, c.NSTG):
        out.ins += pros[s].ins
    out.ins += tail.ins
    return out.ins


def operand_lists(c: Config):
    outs = [("cnt", "+s"), ("tok", "+v")]
    for n in ("q", "do", "lse", "del"):
        outs.append((f"p{n}", f"+{{s[{PTR_SGPR[n]}:{PTR_SGPR[n] + 1}]}}"))
    for n in TEMP_SGPRS:
        outs.append((n, "=&s"))
    ins = []
    for blk in range(c.CB):
        for j in range(c.NJ):
            ins.append((f"k{blk}_{j}", "v"))
    for j in range(c.NJ):
        ins.append((f"qrow{j}", "v"))
    for db in range(c.DB):
        for sx in range(1 if c.half_affine else 2):
            for w in range(2):
                ins.append((f"qtr{db}_{w}" if c.half_affine else f"qtr{db}_{sx}_{w}", "v"))
    for j in range(c.NJ):
        ins.append((f"vrow{j}", "v"))
    for n in ["vec"] + [f"g{t}{i}" for t in ("q", "do") for i in range(c.slabs)] + ["lane4"]:
        ins.append((n, "v"))
    for n in ("scale", "dmabase", "vecdma", "qstep", "dostep", "vecwave", "st0", "tailn"):
        ins.append((n, "s"))
    # the vector registers of the statement's own, and the accumulation registers of dV^T and dK^T (which
    # the kernel names itself everywhere: the compiler keeps out of them)
    clob = [f"v{r}" for r in range(c.nvgpr)] + [f"a{r}" for r in range(2 * c.CB * c.DB * 16)]
    return outs, ins, clob


def emit_macro(c: Config, out):
    ins = gen_statement(c)
    outs, inputs, clob = operand_lists(c)
    check_clobbers(ins, outs, clob + SPECIAL_CLOBBERS, c.name)
    names = [n for n, _ in outs if n not in TEMP_SGPRS] + [n for n, _ in inputs]
    n_mfma = sum(1 for i in ins if i["kind"] == "mfma")
    out.write(f"// {c.name}: {c.elem} D={c.D}; {c.nvgpr} vector registers of its own, {len(ins)} instructions, "
              f"{n_mfma} MFMAs\n")
    out.write(f"#define {c.name}_VGPRS {c.nvgpr}\n")
    out.write(f"#define {c.name}({', '.join('A_' + n for n in names)}) \\\n")
    out.write("    do { unsigned long long t_ex_; asm volatile( \\\n")
    for i in ins:
        out.write(f'        "{i["text"]}\\n\\t" \\\n')
    tmpmap = {"execsave": "t_ex_"}
    o_s = ", ".join(f'[{n}] "{cs}"({tmpmap.get(n, "A_" + n)})' for n, cs in outs)
    i_s = ", ".join(f'[{n}] "{cs}"(A_{n})' for n, cs in inputs)
    c_s = ", ".join(f'"{x}"' for x in ["memory"] + SPECIAL_CLOBBERS + clob)
    out.write(f"        : {o_s} \\\n        : {i_s} \\\n        : {c_s}); }} while (0)\n\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("-o", "--output", default="chill_bwd_loop.inc")
    ap.add_argument("--barrier-slot", type=int, default=None, help="timing experiments: slot of the early barrier")
    ap.add_argument("--units", type=int, default=None, help="timing experiments: ring units")
    ap.add_argument("--split-a", type=int, default=None, help="timing experiments: S_0 before S_1")
    ap.add_argument("--ablate", default="", help="timing experiments: comma-separated parts to leave out "
                                                 "(barrier, valu, lds, dma, mfma); the results are wrong")
    args = ap.parse_args()
    ABLATE.update(x for x in args.ablate.split(",") if x)
    with open(args.output, "w") as out:
        out.write("// Generated by gen_bwd_loop.py; do not edit.\n#pragma once\n\n")
        if ABLATE:
            out.write("#ifndef CHILL_TIMING_EXPERIMENT\n#error \"a loop with parts left out (--ablate): timing experiments only\"\n#endif\n\n")
        kw = {k: v for k, v in (("barrier_slot", args.barrier_slot), ("units", args.units), ("split_a", args.split_a)) if v is not None}
        for D in (128, 64):
            for c in (Config("bf16", D, **kw), Config("f16", D, **kw)):
                emit_macro(c, out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
