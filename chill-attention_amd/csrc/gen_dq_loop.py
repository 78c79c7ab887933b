#!/usr/bin/env python3
"""Generates the hand-scheduled inner loop of the dQ kernel with register-resident Q and dO
(chill_bwd_dq_gen.h, two 32-row query blocks per wave) as an inline-asm statement: chill_dq_loop.inc,
one macro per element type.

One wave of a 4-wave workgroup (one wave per SIMD) owns 64 query rows: Q and dO as MFMA B operands
and the dQ^T accumulators (2 x D/32 blocks) in the accumulation registers.  An ITERATION takes one
32-key tile of K and V from a ring of four LDS stages; every operand read from LDS feeds two MFMAs
(one per query block).  Reference: chill_attention/chill_bwd_dq.py:262-303.

    A_k  16 MFMAs   S_c^T  = K_k Q_c^T                     (c = 0, 1: the wave's two query blocks)
    B_k  16 MFMAs   dP'_c^T = V_k dO_c^T - delta_c          (the chain starts from a block filled with -delta_c)
    C_k  16 MFMAs   dQ_c^T += K_k^T dS_c^T                  dS = P o dP',  P = exp2(S * scale - LSE2_c)

The loop is software-pipelined over the tiles: an iteration runs A_k, then C_(k-1), then B_k.  The vector
work of tile k-1 that C needs (dS, packed) rides under A_k, the exponentials of tile k under C_(k-1) and
B_k: about two vector instructions per MFMA everywhere.  S is double-buffered by the parity of the tile.
The K rows of tile k+1 are read at the end of iteration k; the barrier of the iteration stands in front of
B_k, where every read of tile k-1 has returned: the tile three ahead is issued into its stage behind it.

The statement runs `cnt` consecutive iterations of one wave: a first one without C, `cnt - 1` of the steady
kind, and the tail (dS and C of the last tile).  The caller guarantees that every tile of the run is
predicate-free for the wave's 64 rows and that the tiles the run issues exist in full.
"""
from __future__ import annotations

import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from asm_stream import AGPR, Sched, Stream, areg, check_clobbers, check_stream, deal, rng, vr  # noqa: E402

PTR_SGPR = {"k": 88, "v": 90}
SPECIAL_CLOBBERS = ["vcc", "scc", "m0"]


class Config:
    def __init__(self, elem: str, D: int = 128, pool: int = 6):
        assert elem in ("bf16", "f16") and D == 128
        self.elem, self.D = elem, D
        self.CB, self.NSTG, self.NW = 2, 4, 4
        self.NJ = D // 16
        self.DB = D // 32
        self.row_bytes = 2 * D
        self.tile = 32 * self.row_bytes   # a 32-key tile of K or of V
        self.stage = 2 * self.tile        # K, then V
        self.pool = pool                  # ring units besides the eight that hold the K rows of a tile
        r = 0
        self.S = ((r, r + 16), (r + 32, r + 48)); r += 64     # S[parity][block]
        self.DP = (r, r + 16); r += 32
        self.PB = (r, r + 8); r += 16
        self.RING = r; r += 4 * (self.NJ + pool)
        self.T = r; r += 4
        self.nvgpr = r
        self.mfma = "v_mfma_f32_32x32x16_" + elem
        self.cvt = "v_cvt_pk_bf16_f32" if elem == "bf16" else "v_cvt_pk_f16_f32"
        self.name = f"CHILL_DQ_LOOP_{elem.upper()}_{D}"
        self.loads_per_tile = 4           # per wave: two slabs of K, two of V
        # accumulation registers: dQ^T block (c, db), then the resident Q and dO chunks (c, j)
        self.n_acc = self.CB * self.DB * 16

    def dq(self, c, db):
        return AGPR + 16 * (c * self.DB + db)

    def qreg(self, c, j):
        return AGPR + self.n_acc + 4 * (c * self.NJ + j)

    def doreg(self, c, j):
        return AGPR + self.n_acc + 4 * self.CB * self.NJ + 4 * (c * self.NJ + j)

    def unit(self, u):
        return self.RING + 4 * u


def exp_ops(c: Config, st: Stream, par: int, blk: int):
    """P = exp2(S * scale - LSE2), in place."""
    S = c.S[par][blk]
    ops = []
    for k in range(8):
        t0, t1 = c.T + (2 * k) % 4, c.T + (2 * k + 1) % 4
        for e, t in ((2 * k, t0), (2 * k + 1, t1)):
            ops.append(lambda e=e, t=t: st.add(f"v_fma_f32 {vr(t)}, {vr(S + e)}, %[scale], -%[lse{blk}]", "valu", [S + e], [t]))
        for e, t in ((2 * k, t0), (2 * k + 1, t1)):
            ops.append(lambda e=e, t=t: st.add(f"v_exp_f32 {vr(S + e)}, {vr(t)}", "trans", [t], [S + e]))
    return ops


def grad_ops(c: Config, st: Stream, par: int, half: int):
    """dS = P o dP' for entries 8 * half .. 8 * half + 7 of both blocks, packed into PB[block][4 * half ..]."""
    ops = []
    for blk in range(c.CB):
        S, DP = c.S[par][blk], c.DP[blk]
        for e in range(8 * half, 8 * half + 8):
            ops.append(lambda e=e, S=S, DP=DP: st.add(f"v_mul_f32 {vr(DP + e)}, {vr(S + e)}, {vr(DP + e)}", "valu",
                                                      [S + e, DP + e], [DP + e]))
    for blk in range(c.CB):
        DP, PB = c.DP[blk], c.PB[blk]
        for k in range(4 * half, 4 * half + 4):
            ops.append(lambda k=k, DP=DP, PB=PB: st.add(f"{c.cvt} {vr(PB + k)}, {vr(DP + 2 * k)}, {vr(DP + 2 * k + 1)}",
                                                        "valu", [DP + 2 * k, DP + 2 * k + 1], [PB + k]))
    return ops


def dma_ops(c: Config, st: Stream, tgt: int):
    A = st.add
    ops = []
    base = tgt * c.stage
    for name, off in (("k", 0), ("v", c.tile)):
        for i in range(2):
            def load(name=name, off=off, i=i):
                A(f"s_add_u32 m0, %[dmabase], {base + off + i * c.NW * 1024}", "salu")
                A("s_nop 0", "nop")
                A(f"global_load_lds_dwordx4 %[g{name}{i}], s[{PTR_SGPR[name]}:{PTR_SGPR[name] + 1}]", "vmem")
            ops.append(load)
    for name in ("k", "v"):
        lo, hi = f"s{PTR_SGPR[name]}", f"s{PTR_SGPR[name] + 1}"

        def advance(lo=lo, hi=hi, name=name):
            A(f"s_add_u32 {lo}, {lo}, %[{name}step]", "salu")
            A(f"s_addc_u32 {hi}, {hi}, 0", "salu")
        ops.append(advance)
    return ops


def k_row_reads(c: Config, stage: int):
    """The K rows of the tile in `stage` into the units 0 .. NJ-1: (text, registers)."""
    return [(f"ds_read_b128 {vr(c.unit(j), 4)}, %[krow{j}] offset:{stage * c.stage}", rng(c.unit(j), 4)) for j in range(c.NJ)]


def gen_body(c: Config, st: Stream, s: int, first: bool):
    """One iteration for the tile in stage s: A_k, C_(k-1) (not in the first one), barrier, B_k."""
    par = s % 2
    prev, nxt, tgt = (s + 3) % c.NSTG, (s + 1) % c.NSTG, (s + 3) % c.NSTG
    sch = Sched(st, [regs for _, regs in k_row_reads(c, s)])
    slots = [("A", j, blk) for j in range(c.NJ) for blk in range(c.CB)]
    if not first:
        slots += [("C", sx, db, blk) for sx in range(2) for db in range(c.DB) for blk in range(c.CB)]
    b0 = len(slots)   # the barrier stands in front of this slot
    slots += [("B", j, blk) for j in range(c.NJ) for blk in range(c.CB)]
    NS = len(slots)
    last_use = {}
    for t, sl in enumerate(slots):
        last_use[sl[:2] if sl[0] != "C" else sl[:3]] = t
    queue = []
    if not first:
        queue += [(("C", sx, db), 0) for sx in range(2) for db in range(c.DB)]
    queue += [(("B", j), 0) for j in range(c.NJ)]
    queue += [(("N", j), b0) for j in range(c.NJ)]   # the K rows of the next tile: certified by this iteration's barrier
    unit_of = {("A", j): j for j in range(c.NJ)}
    free = list(range(c.NJ, c.NJ + c.pool))

    def read_text(key, u):
        r = c.unit(u)
        if key[0] == "C":
            off = prev * c.stage + key[1] * 16 * c.row_bytes
            return [(f"ds_read_b64_tr_b16 {vr(r, 2)}, %[ktr{key[2]}_0] offset:{off}", rng(r, 2)),
                    (f"ds_read_b64_tr_b16 {vr(r + 2, 2)}, %[ktr{key[2]}_1] offset:{off}", rng(r + 2, 2))]
        if key[0] == "B":
            return [(f"ds_read_b128 {vr(r, 4)}, %[krow{key[1]}] offset:{s * c.stage + c.tile}", rng(r, 4))]
        return [k_row_reads(c, nxt)[key[1]]]

    valu = [[] for _ in range(NS)]

    def place(ops, lo, hi):
        for t, lst in enumerate(deal(ops, lo, hi, NS)):
            valu[t] += lst
    if first:
        place(exp_ops(c, st, par, 0) + exp_ops(c, st, par, 1), 18, NS - 1)
    else:
        place(grad_ops(c, st, par ^ 1, 0), 4, 13)
        place(grad_ops(c, st, par ^ 1, 1), 12, 21)
        place(exp_ops(c, st, par, 0) + exp_ops(c, st, par, 1), 19, NS - 1)
    scalar = deal(dma_ops(c, st, tgt), b0, b0 + 11, NS)
    for t, sl in enumerate(slots):
        if t == b0:
            # every read of the tile before has returned and been used (C is behind us): its stage may be refilled
            assert not any(k[0] == "C" for k, _ in queue)
            st.add(f"s_waitcnt vmcnt({c.loads_per_tile})", "wait")
            st.add("s_barrier", "salu")
        if sl[0] == "A":
            _, j, blk = sl
            a = c.unit(unit_of[("A", j)])
            S = c.S[par][blk]
            sch.need(rng(a, 4))
            b = c.qreg(blk, j)
            st.add(f"{c.mfma} {vr(S, 16)}, {vr(a, 4)}, {areg(b, 4)}, {'0' if j == 0 else vr(S, 16)}", "mfma",
                   rng(a, 4) + ([] if j == 0 else rng(S, 16)), rng(S, 16))
        elif sl[0] == "B":
            _, j, blk = sl
            a = c.unit(unit_of[("B", j)])
            DP = c.DP[blk]
            sch.need(rng(a, 4))
            b = c.doreg(blk, j)
            cin = f"%[nd{blk}]" if j == 0 else vr(DP, 16)
            st.add(f"{c.mfma} {vr(DP, 16)}, {vr(a, 4)}, {areg(b, 4)}, {cin}", "mfma",
                   rng(a, 4) + ([] if j == 0 else rng(DP, 16)), rng(DP, 16))
        else:
            _, sx, db, blk = sl
            a = c.unit(unit_of[("C", sx, db)])
            acc = c.dq(blk, db)
            b = c.PB[blk] + 4 * sx
            sch.need(rng(a, 4))
            st.add(f"{c.mfma} {areg(acc, 16)}, {vr(a, 4)}, {vr(b, 4)}, {areg(acc, 16)}", "mfma",
                   rng(a, 4) + rng(b, 4) + rng(acc, 16), rng(acc, 16))
        for key, last in last_use.items():
            if last == t and key in unit_of:
                u = unit_of.pop(key)
                if u >= c.NJ:
                    free.append(u)
        issued = 0
        while queue and issued < 3:
            key, ready = queue[0]
            if ready > t:
                break
            if key[0] == "N":
                # unit j once more; the K rows of this tile have long been used
                assert ("A", key[1]) not in unit_of
                u = key[1]
            else:
                if not free:
                    break
                u = free.pop(free.index(min(free)))
                unit_of[key] = u
            for text, regs in read_text(key, u):
                sch.read(text, None, regs)
            queue.pop(0)
            issued += 1
        for op in valu[t]:
            op()
        for op in scalar[t]:
            op()
    assert not queue, f"reads left over: {queue}"


def gen_tail(c: Config, st: Stream, s: int):
    """dS and C of the last tile of a run (stage s)."""
    par = s % 2
    sch = Sched(st)
    st.add("s_waitcnt lgkmcnt(0)", "wait", wait=0)   # the K rows read ahead for an iteration that the caller runs
    st.add("s_nop 7", "nop", nops=8)                # the last dP' may still be in the matrix pipe
    for sx in range(2):
        for db in range(c.DB):
            r = c.unit(sx * c.DB + db)
            off = s * c.stage + sx * 16 * c.row_bytes
            sch.read(f"ds_read_b64_tr_b16 {vr(r, 2)}, %[ktr{db}_0] offset:{off}", None, rng(r, 2))
            sch.read(f"ds_read_b64_tr_b16 {vr(r + 2, 2)}, %[ktr{db}_1] offset:{off}", None, rng(r + 2, 2))
    for half in range(2):
        for op in grad_ops(c, st, par, half):
            op()
    st.add("s_nop 1", "nop", nops=2)
    for sx in range(2):
        for db in range(c.DB):
            for blk in range(c.CB):
                a = c.unit(sx * c.DB + db)
                acc = c.dq(blk, db)
                b = c.PB[blk] + 4 * sx
                sch.need(rng(a, 4))
                st.add(f"{c.mfma} {areg(acc, 16)}, {vr(a, 4)}, {vr(b, 4)}, {areg(acc, 16)}", "mfma",
                       rng(a, 4) + rng(b, 4) + rng(acc, 16), rng(acc, 16))


def gen_statement(c: Config):
    S = Stream
    out = S()
    A = out.add
    for s in range(1, c.NSTG):
        A(f"s_cmp_eq_u32 %[st0], {s}", "salu")
        A(f"s_cbranch_scc1 .Lfirst{s}%=", "salu")
    firsts, bodies, tails = [], [], []
    for s in range(c.NSTG):
        f = S()
        f.add(f".Lfirst{s}%=:", "label", nops=0)
        # (the tile has been certified by the barrier of the iteration before, which the caller ran)
        sch = Sched(f)
        for text, regs in k_row_reads(c, s):
            sch.read(text, None, regs)
        gen_body(c, f, s, first=True)
        f.add("s_sub_u32 %[cnt], %[cnt], 1", "salu")
        f.add("s_cmp_eq_u32 %[cnt], 0", "salu")
        f.add(f"s_cbranch_scc1 .Ltail{s}%=", "salu")
        f.add(f"s_branch .Lbody{(s + 1) % c.NSTG}%=", "salu")
        firsts.append(f)
        b = S()
        b.add(f".Lbody{s}%=:", "label", nops=0)
        gen_body(c, b, s, first=False)
        b.add("s_sub_u32 %[cnt], %[cnt], 1", "salu")
        b.add("s_cmp_eq_u32 %[cnt], 0", "salu")
        b.add(f"s_cbranch_scc1 .Ltail{s}%=", "salu")
        if s == c.NSTG - 1:
            b.add("s_branch .Lbody0%=", "salu")
        bodies.append(b)
        t = S()
        t.add(f".Ltail{s}%=:", "label", nops=0)
        gen_tail(c, t, s)
        t.add("s_branch .Lend%=", "salu")
        tails.append(t)
    for s in range(c.NSTG):
        n1, n2 = (s + 1) % c.NSTG, (s + 2) % c.NSTG
        check_stream(firsts[s].ins + tails[s].ins, f"{c.name} (one iteration, stage {s})")
        check_stream(firsts[s].ins + bodies[n1].ins + bodies[n2].ins + tails[n2].ins, f"{c.name} (from stage {s})")
        check_stream(firsts[s].ins + bodies[n1].ins + tails[n1].ins, f"{c.name} (two iterations from stage {s})")
    out.ins += firsts[0].ins
    for s in range(c.NSTG):
        out.ins += bodies[s].ins
    for s in range(1, c.NSTG):
        out.ins += firsts[s].ins
    for s in range(c.NSTG):
        out.ins += tails[s].ins
    out.add(".Lend%=:", "label", nops=0)
    out.add("s_nop 7", "nop", nops=8)
    return out.ins


def operand_lists(c: Config):
    outs = [("cnt", "+s"), ("tok", "+v")]
    for n in ("k", "v"):
        outs.append((f"p{n}", f"+{{s[{PTR_SGPR[n]}:{PTR_SGPR[n] + 1}]}}"))
    ins = [("nd0", "v"), ("nd1", "v"), ("lse0", "v"), ("lse1", "v")]
    for j in range(c.NJ):
        ins.append((f"krow{j}", "v"))
    for db in range(c.DB):
        for w in range(2):
            ins.append((f"ktr{db}_{w}", "v"))
    for n in ("gk0", "gk1", "gv0", "gv1"):
        ins.append((n, "v"))
    for n in ("scale", "dmabase", "kstep", "vstep", "st0"):
        ins.append((n, "s"))
    # its own vector registers, and every accumulation register: the dQ^T accumulators, which it writes, and the resident
    # Q and dO behind them, which it only reads -- named here so that the compiler parks nothing in them across the
    # statement (the kernel names all 256 itself; what the compiler does with them elsewhere is checked on the assembly)
    clob = [f"v{r}" for r in range(c.nvgpr)] + [f"a{r}" for r in range(256)]
    return outs, ins, clob


def emit_macro(c: Config, out):
    ins = gen_statement(c)
    outs, inputs, clob = operand_lists(c)
    check_clobbers(ins, outs, clob + SPECIAL_CLOBBERS, c.name)
    names = [n for n, _ in outs] + [n for n, _ in inputs]
    n_mfma = sum(1 for i in ins if i["kind"] == "mfma")
    out.write(f"// {c.name}: {c.elem} D={c.D}; {c.nvgpr} vector registers of its own, {len(ins)} instructions, "
              f"{n_mfma} MFMAs\n")
    out.write(f"#define {c.name}_VGPRS {c.nvgpr}\n")
    out.write(f"#define {c.name}({', '.join('A_' + n for n in names)}) \\\n")
    out.write("    do { asm volatile( \\\n")
    for i in ins:
        out.write(f'        "{i["text"]}\\n\\t" \\\n')
    o_s = ", ".join(f'[{n}] "{cs}"(A_{n})' for n, cs in outs)
    i_s = ", ".join(f'[{n}] "{cs}"(A_{n})' for n, cs in inputs)
    c_s = ", ".join(f'"{x}"' for x in ["memory"] + SPECIAL_CLOBBERS + clob)
    out.write(f"        : {o_s} \\\n        : {i_s} \\\n        : {c_s}); }} while (0)\n\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("-o", "--output", default="chill_dq_loop.inc")
    args = ap.parse_args()
    with open(args.output, "w") as out:
        out.write("// Generated by gen_dq_loop.py; do not edit.\n#pragma once\n\n")
        for c in (Config("bf16"), Config("f16")):
            emit_macro(c, out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
