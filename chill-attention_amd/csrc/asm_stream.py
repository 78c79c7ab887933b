"""Instruction streams for the generated inner loops (gen_fwd_loop.py, gen_bwd_loop.py): the list of
instructions with what each reads and writes, and the checks a hand-written gfx950 stream has to pass
because no compiler sees it: data hazards between the matrix pipe, the vector ALU and LDS reads
(check_stream), and the operand and clobber lists of the inline-asm statement (check_clobbers).

Registers are numbered: vector registers by their index, accumulation registers by AGPR + index.
"""
from __future__ import annotations

AGPR = 1000             # register number of a0 in the bookkeeping

LGKM_MAX = 15           # the counter of outstanding LDS operations has four bits
MFMA_RESULT_WAIT = 11   # wait states before a non-MFMA instruction may read an 8-pass MFMA result
VALU_TO_MFMA_WAIT = 2   # wait states between a VALU write and an MFMA that reads the register
TRANS_USE_WAIT = 1      # wait states between v_exp_f32 and a VALU read of its result


def vr(base, n=1):
    return f"v{base}" if n == 1 else f"v[{base}:{base + n - 1}]"


def rng(base, n):
    return list(range(base, base + n))


class Stream:
    """Instruction list with the bookkeeping check_stream needs."""

    def __init__(self):
        self.ins = []

    def add(self, text, kind, reads=(), writes=(), nops=1, lds=False, wait=None):
        self.ins.append(dict(text=text, kind=kind, reads=set(reads), writes=set(writes), nops=nops, lds=lds,
                             wait=wait))


def check_stream(ins, what):
    """Hazards of a straight-line instruction stream.  LDS reads complete in order; `wait` = the
    lgkmcnt operand of an s_waitcnt.  Positions are counted in wait states."""
    pending = {}            # vgpr -> sequence number of the LDS read that will write it
    issued = 0              # LDS reads issued so far
    last_mfma_write, last_valu_write, last_trans_write = {}, {}, {}
    pos = 0
    for i in ins:
        k = i["kind"]
        if k == "wait" and i["wait"] is not None:
            done_upto = issued - i["wait"]
            for reg in [r for r, s in pending.items() if s <= done_upto]:
                del pending[reg]
        for reg in i["reads"] | i["writes"]:
            if reg in pending:
                raise SystemExit(f"{what}: '{i['text']}' touches v{reg} while an LDS read into it is in flight")
        if k == "mfma":
            for reg in i["reads"]:
                if reg in last_valu_write and pos - last_valu_write[reg] - 1 < VALU_TO_MFMA_WAIT:
                    raise SystemExit(f"{what}: '{i['text']}' reads v{reg} too soon after a VALU write")
                if reg in last_mfma_write and reg not in i["writes"] and pos - last_mfma_write[reg] - 1 < MFMA_RESULT_WAIT:
                    raise SystemExit(f"{what}: '{i['text']}' reads MFMA result v{reg} as A/B too soon")
        elif k in ("valu", "trans", "lds"):
            for reg in i["reads"]:
                if reg in last_mfma_write and pos - last_mfma_write[reg] - 1 < MFMA_RESULT_WAIT:
                    raise SystemExit(f"{what}: '{i['text']}' reads MFMA result v{reg} after "
                                     f"{pos - last_mfma_write[reg] - 1} wait states")
                if k != "lds" and reg in last_trans_write and pos - last_trans_write[reg] - 1 < TRANS_USE_WAIT:
                    raise SystemExit(f"{what}: '{i['text']}' reads v{reg} right after v_exp_f32")
            if k != "lds":
                for reg in i["writes"]:
                    if reg in last_mfma_write and pos - last_mfma_write[reg] - 1 < MFMA_RESULT_WAIT:
                        raise SystemExit(f"{what}: '{i['text']}' overwrites v{reg} under a running MFMA")
        if i["lds"]:
            issued += 1
            for reg in i["writes"]:
                pending[reg] = issued
        for reg in i["writes"]:
            if k == "mfma":
                last_mfma_write[reg] = pos
                last_valu_write.pop(reg, None)
                last_trans_write.pop(reg, None)
            elif k in ("valu", "trans"):
                last_valu_write[reg] = pos
                last_mfma_write.pop(reg, None)
                if k == "trans":
                    last_trans_write[reg] = pos
                else:
                    last_trans_write.pop(reg, None)
            elif k == "lds":
                last_mfma_write.pop(reg, None)
                last_valu_write.pop(reg, None)
                last_trans_write.pop(reg, None)
        pos += i["nops"]
    if pending:
        raise SystemExit(f"{what}: LDS reads still in flight at the end")


def check_clobbers(ins, outs, clobbers, what):
    """Everything the statement writes is an output operand or a clobber: vector registers from the
    bookkeeping of the stream, scalar destinations from the text (named operands %[x] must be outputs;
    physical and special registers must be clobbers or tied output registers)."""
    import re

    out_names = {n for n, _ in outs}
    out_regs = set()
    for _, cs in outs:
        m = re.search(r"\{v\[(\d+):(\d+)\]\}", cs)
        if m:
            out_regs |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        m = re.search(r"\{v(\d+)\}", cs)
        if m:
            out_regs.add(int(m.group(1)))
    out_sregs = set()
    for _, cs in outs:
        m = re.search(r"\{s\[(\d+):(\d+)\]\}", cs)
        if m:
            out_sregs |= {f"s{r}" for r in range(int(m.group(1)), int(m.group(2)) + 1)}
    clob_v = {int(x[1:]) for x in clobbers if re.fullmatch(r"v\d+", x)}
    clob_v |= {AGPR + int(x[1:]) for x in clobbers if re.fullmatch(r"a\d+", x)}
    for i in ins:
        for reg in i["writes"]:
            if reg not in out_regs and reg not in clob_v:
                name = f"a{reg - AGPR}" if reg >= AGPR else f"v{reg}"
                raise SystemExit(f"{what}: '{i['text']}' writes {name}, which is neither an output nor a clobber")
        if i["kind"] != "salu" and not i["text"].startswith("v_cmp"):
            continue
        parts = i["text"].split(None, 1)
        if len(parts) < 2 or parts[0] in ("s_barrier", "s_branch", "s_nop") or parts[0].startswith("s_cbranch"):
            continue
        dest = parts[1].split(",")[0].strip()
        if parts[0].startswith("s_cmp"):
            dest = "scc"
        m = re.fullmatch(r"%\[(\w+)\]", dest)
        if m:
            if m.group(1) not in out_names:
                raise SystemExit(f"{what}: '{i['text']}' writes the input operand {dest}")
            continue
        if dest == "exec":
            continue  # saved at the head of the statement and restored by every instruction that changes it
        if dest not in clobbers and dest not in out_sregs:
            raise SystemExit(f"{what}: '{i['text']}' writes {dest}, which is neither an output nor a clobber")
        # instructions that set SCC as a side effect
        if re.match(r"s_(add|sub|addc|and|or)", parts[0]) and "scc" not in clobbers:
            raise SystemExit(f"{what}: '{i['text']}' sets SCC, which is not a clobber")
    # EXEC: saved before its first change, and every change is followed by a restore
    saved = restored = True
    for i in ins:
        t = i["text"]
        if t == "s_mov_b64 %[execsave], exec":
            if not restored:
                raise SystemExit(f"{what}: EXEC is saved while it is changed")
            saved_once = True
        elif t.startswith("s_mov_b64 exec"):
            if "saved_once" not in locals():
                raise SystemExit(f"{what}: EXEC is changed without being saved and restored")
            restored = t == "s_mov_b64 exec, %[execsave]"
    if not restored:
        raise SystemExit(f"{what}: EXEC is changed without being saved and restored")


def areg(base, n):
    b = base - AGPR
    return f"a[{b}:{b + n - 1}]"


class Sched:
    """Emits into a Stream, keeps the order of the LDS reads and computes the waits."""

    def __init__(self, st: Stream, carried=()):
        self.st = st
        self.seq = 0
        self.pending = {}
        for regs in carried:      # reads of the iteration before that may still be in flight, oldest first
            self.seq += 1
            for r in regs:
                self.pending[r] = self.seq

    def read(self, text, addr, regs):
        self.st.add(text, "lds", [], regs, lds=True)
        self.seq += 1
        for r in regs:
            self.pending[r] = self.seq

    def need(self, regs):
        seqs = [self.pending[r] for r in regs if r in self.pending]
        if not seqs:
            return
        last = max(seqs)
        n = min(self.seq - last, LGKM_MAX)
        self.st.add(f"s_waitcnt lgkmcnt({n})", "wait", wait=n)
        done = self.seq - n
        for r in [r for r, s in self.pending.items() if s <= done]:
            del self.pending[r]

    def wait_upto(self, seq):
        """All reads up to sequence number `seq` have returned."""
        n = min(self.seq - seq, LGKM_MAX)
        if any(s <= seq for s in self.pending.values()):
            self.st.add(f"s_waitcnt lgkmcnt({n})", "wait", wait=n)
            done = self.seq - n
            for r in [r for r, s in self.pending.items() if s <= done]:
                del self.pending[r]

    def wait_all(self):
        self.st.add("s_waitcnt lgkmcnt(0)", "wait", wait=0)
        self.pending.clear()


def deal(ops, lo, hi, nslots):
    """ops dealt evenly over slots lo .. hi (inclusive), in order."""
    share = [[] for _ in range(nslots)]
    n = hi - lo + 1
    for i, op in enumerate(ops):
        share[lo + i * n // len(ops)].append(op)
    return share
