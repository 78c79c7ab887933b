"""The generator of the forward's hand-scheduled loop (csrc/gen_fwd_loop.py): every configuration it ships
passes its own hazard check, and the check catches the mistakes it exists for."""

import importlib.util
import io
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_spec = importlib.util.spec_from_file_location(
    "gen_fwd_loop", os.path.join(ROOT, "chill-attention_amd", "csrc", "gen_fwd_loop.py"))
gen = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(gen)

_spec_b = importlib.util.spec_from_file_location(
    "gen_bwd_loop", os.path.join(ROOT, "chill-attention_amd", "csrc", "gen_bwd_loop.py"))
genb = importlib.util.module_from_spec(_spec_b)
_spec_b.loader.exec_module(genb)

CONFIGS = [("bf16", 128, 8, 4), ("f16", 128, 8, 4), ("bf16", 64, 4, 3), ("f16", 64, 4, 3)]


@pytest.mark.parametrize("elem,D,waves,stages", CONFIGS)
def test_configurations_generate_and_pass_the_hazard_check(elem, D, waves, stages):
    c = gen.Config(elem, D, waves, stages)
    out = io.StringIO()
    gen.emit_macro(c, out)  # raises SystemExit if a hazard rule is broken
    text = out.getvalue()
    assert f"#define {c.name}(" in text and c.nvgpr <= 256
    # one MFMA per slot: a 64-key tile of the steady state holds 2 steps x 2 phases x D / 16 of them
    assert text.count("v_mfma_f32_32x32x16_" + elem) % (D // 16) == 0
    # every LDS read is waited for by a counted s_waitcnt, never by a blanket one inside the loop body
    assert "lgkmcnt(" in text


def _stream(*ins):
    st = gen.Stream()
    for kind, text, reads, writes, kw in ins:
        st.add(text, kind, reads, writes, **kw)
    return st.ins


def test_check_catches_an_early_read_of_an_mfma_result():
    mfma = ("mfma", "v_mfma v[0:15], v[16:19], v[20:23], v[0:15]", list(range(16, 24)) + list(range(16)), list(range(16)), {})
    use = ("valu", "v_exp_f32 v30, v0", [0], [30], {})
    nop = ("nop", "s_nop 7", [], [], {"nops": 8})
    with pytest.raises(SystemExit, match="reads MFMA result"):
        gen.check_stream(_stream(mfma, use), "early read")
    gen.check_stream(_stream(mfma, nop, nop, use), "late enough")


def test_check_catches_a_register_with_an_lds_read_in_flight():
    read = ("lds", "ds_read_b128 v[16:19], v40", [40], [16, 17, 18, 19], {"lds": True})
    mfma = ("mfma", "v_mfma v[0:15], v[16:19], v[20:23], v[0:15]", list(range(16, 24)) + list(range(16)), list(range(16)), {})
    wait = ("wait", "s_waitcnt lgkmcnt(0)", [], [], {"wait": 0})
    with pytest.raises(SystemExit, match="LDS read into it is in flight"):
        gen.check_stream(_stream(read, mfma), "no wait")
    gen.check_stream(_stream(read, wait, mfma), "waited")
    # a wait that leaves the newest read outstanding does not cover it
    with pytest.raises(SystemExit, match="in flight"):
        gen.check_stream(_stream(read, ("wait", "s_waitcnt lgkmcnt(1)", [], [], {"wait": 1}), mfma), "short wait")


def test_check_catches_a_vector_write_right_before_its_mfma():
    write = ("valu", "v_cvt_pk_bf16_f32 v20, v30, v31", [30, 31], [20], {})
    mfma = ("mfma", "v_mfma v[0:15], v[16:19], v[20:23], v[0:15]", list(range(16, 24)) + list(range(16)), list(range(16)), {})
    with pytest.raises(SystemExit, match="too soon after a VALU write"):
        gen.check_stream(_stream(write, mfma), "no wait states")
    gen.check_stream(_stream(write, ("nop", "s_nop 1", [], [], {"nops": 2}), mfma), "two wait states")


@pytest.mark.parametrize("elem,D,waves,stages", CONFIGS)
def test_statement_declares_everything_it_writes(elem, D, waves, stages):
    """The clobber list and the output operands of the generated statement cover every register its
    instructions write (M0, VCC and SCC among them), and EXEC is saved and restored."""
    c = gen.Config(elem, D, waves, stages)
    ins = gen.gen_loop(c)
    outs, inputs, clob = gen.operand_lists(c)
    gen.check_clobbers(ins, outs, clob + gen.SPECIAL_CLOBBERS, c.name)
    assert "m0" in gen.SPECIAL_CLOBBERS and any(i["text"].startswith("s_add_u32 m0") for i in ins)
    # a list without M0, or without one of the scratch registers, is refused
    with pytest.raises(SystemExit, match="writes m0"):
        gen.check_clobbers(ins, outs, clob + ["vcc", "scc"], c.name)
    with pytest.raises(SystemExit, match="neither an output nor a clobber"):
        gen.check_clobbers(ins, outs, clob[1:] + gen.SPECIAL_CLOBBERS, c.name)
    # so is a write to an input operand
    bad = list(ins) + [dict(text="s_mov_b32 %[lds0], 0", kind="salu", reads=set(), writes=set(), nops=1, lds=False, wait=None)]
    with pytest.raises(SystemExit, match="writes the input operand"):
        gen.check_clobbers(bad, outs, clob + gen.SPECIAL_CLOBBERS, c.name)
    # and an EXEC that is set without having been saved
    unsaved = [i for i in ins if i["text"] != "s_mov_b64 %[execsave], exec"]
    with pytest.raises(SystemExit, match="EXEC is changed"):
        gen.check_clobbers(unsaved, outs, clob + gen.SPECIAL_CLOBBERS, c.name)


@pytest.mark.parametrize("elem", ["bf16", "f16"])
def test_backward_loop_at_head_dim_64(elem):
    """The same generator at head dim 64: half the slots (32 MFMAs per iteration for the same vector work), one slab of a
    tile per wave, and per-lane addresses of their own for the transposed operands of the two 16-row halves of a tile
    (rows of 128 bytes: rows 16 apart do not share the swizzle key).  Every path passes the hazard check."""
    c = genb.Config(elem, 64)
    ins = genb.gen_statement(c)
    outs, inputs, clob = genb.operand_lists(c)
    genb.check_clobbers(ins, outs, clob + genb.SPECIAL_CLOBBERS, c.name)
    names = [n for n, _ in inputs]
    assert [n for n in names if n.startswith("qtr")] == [f"qtr{db}_{sx}_{w}" for db in range(2) for sx in range(2) for w in range(2)]
    assert [n for n in names if n.startswith("g")] == ["gq0", "gdo0"] and sum(n.startswith("k") for n in names) == 8
    cycle, orders = genb.find_steady_state(c)
    it = genb.SteadyIteration(c, cycle[0], orders[-1])
    st = genb.Stream()
    it.generate(st, 0)
    text = [i["text"] for i in st.ins]
    assert sum(t.startswith("v_mfma") for t in text) == 32 and sum(t.startswith("v_exp_f32") for t in text) == 32
    assert sum(t.startswith("ds_read_b128") for t in text) == 4 + 4 + 8 + 4 + 8 and sum(t.startswith("ds_read_b64_tr_b16") for t in text) == 16
    assert sum(t.startswith("global_load_lds_dwordx4") for t in text) == 2
    # no transposed read adds a half-tile offset to its address
    tr = [t for t in text if t.startswith("ds_read_b64_tr_b16")]
    assert all(int(t.split("offset:")[1]) % c.stage in (0, c.tile) for t in tr)
    assert f"s_waitcnt vmcnt({c.loads_per_tile})" in text and c.loads_per_tile == 2


@pytest.mark.parametrize("elem", ["bf16", "f16"])
def test_backward_loop_generates_and_declares_what_it_writes(elem):
    """The generated loop of the dK/dV kernel with register-resident K (csrc/gen_bwd_loop.py): every path through the
    statement (prologue of each stage, its iteration, the next ones, the exit) passes the hazard check, the ring of
    operand registers comes back to where it started after the four unrolled stages, every register it writes is an
    output or a clobber, and an iteration holds the 64 MFMAs and the LDS reads it is meant to."""
    c = genb.Config(elem)
    ins = genb.gen_statement(c)  # raises SystemExit if a hazard rule is broken or the ring does not close
    outs, inputs, clob = genb.operand_lists(c)
    genb.check_clobbers(ins, outs, clob + genb.SPECIAL_CLOBBERS, c.name)
    with pytest.raises(SystemExit, match="neither an output nor a clobber"):
        genb.check_clobbers(ins, outs, [x for x in clob if x != "a17"] + genb.SPECIAL_CLOBBERS, c.name)
    cycle, orders = genb.find_steady_state(c)
    assert c.NSTG % len(cycle) == 0 and c.nvgpr + 64 + 32 <= 256  # its own registers, K, addresses
    it = genb.SteadyIteration(c, cycle[0], orders[-1])
    st = genb.Stream()
    assert it.generate(st, 0) == cycle[1 % len(cycle)]
    text = [i["text"] for i in st.ins]
    mf = [t for t in text if t.startswith("v_mfma")]
    assert len(mf) == 64 and all(elem in t for t in mf)
    # 32 of them accumulate into the sixteen dV^T / dK^T blocks in accumulation registers, each block exactly twice
    acc = [t.split()[1].rstrip(",") for t in mf if t.split()[1].startswith("a[")]
    assert len(acc) == 32 and all(acc.count(a) == 2 for a in set(acc)) and len(set(acc)) == 16
    # LDS: 8 Q + 8 dO + 16 V row chunks, 16 transposed operands of two reads each, LSE2 and twice delta of the next tile
    assert sum(t.startswith("ds_read_b128") for t in text) == 8 + 8 + 16 + 4 + 8
    assert sum(t.startswith("ds_read_b64_tr_b16") for t in text) == 32
    # vector work: 32 exponentials, 32 + 32 multiply(-add)s, 32 packs; four tile loads (and the two of the vectors)
    assert sum(t.startswith("v_exp_f32") for t in text) == 32 and sum(t.startswith("v_fma_f32") for t in text) == 32
    assert sum(t.startswith("v_mul_f32") for t in text) == 32 and sum(t.startswith(c.cvt) for t in text) == 32
    assert sum(t.startswith("global_load_lds_dwordx4") for t in text) == 4 and sum(t.startswith("global_load_lds_dword ") for t in text) == 2
    # every prefetched operand of the next iteration comes from the next stage
    nxt = [t for t in text if "offset:" in t and int(t.split("offset:")[1]) >= c.stage and "%[vrow" not in t]
    assert len(nxt) == 4 + 8 + 8


def test_backward_loop_tail_requests_no_tile():
    """The iterations a run ends with when it reaches the workgroup's last tile (the tiles three ahead do not exist):
    the same 64 MFMAs, LDS reads and vector work, no tile load and no pointer moved on, and the barrier waits for
    every tile still on its way.  The statement holds one such body per stage and enters them by the count."""
    c = genb.Config("bf16")
    cycle, orders = genb.find_steady_state(c)
    it = genb.SteadyIteration(c, cycle[0], orders[-1])
    body, tail = genb.Stream(), genb.Stream()
    assert it.generate(body, 0) == it.generate(tail, 0, with_dma=False)
    kinds = lambda st, k: [i["text"] for i in st.ins if i["kind"] == k]  # noqa: E731
    assert kinds(body, "mfma") == kinds(tail, "mfma") and kinds(body, "valu") == kinds(tail, "valu")
    assert [t for t in kinds(body, "lds")] == [t for t in kinds(tail, "lds")]
    text = [i["text"] for i in tail.ins]
    assert not any("global_load" in t or "s_add_u32" in t or "s_addc_u32" in t for t in text)
    assert "s_waitcnt vmcnt(0)" in text and f"s_waitcnt vmcnt({c.loads_per_tile})" not in text
    assert f"s_waitcnt vmcnt({c.loads_per_tile})" in [i["text"] for i in body.ins]
    # (the padding keeps the distance between the score MFMAs and the vector work that reads them)
    assert sum(i["nops"] for i in tail.ins) >= sum(i["nops"] for i in body.ins) - 4
    whole = [i["text"] for i in genb.gen_statement(c)]
    for s in range(c.NSTG):
        assert f".Ltbody{s}%=:" in whole and f".Ltsel{s}%=:" in whole
    assert whole.count("s_cmp_le_u32 %[cnt], %[tailn]") == 2 * c.NSTG
    assert ("tailn", "s") in genb.operand_lists(c)[1]


def test_backward_loop_check_catches_a_missing_wait():
    """The same stream with one of its computed waits removed does not pass."""
    c = genb.Config("bf16")
    cycle, orders = genb.find_steady_state(c)
    it = genb.SteadyIteration(c, cycle[0], orders[-1])
    pro, st = genb.Stream(), genb.Stream()
    sch = genb.Sched(pro)
    for text, regs in it.reads_for_stage(0):
        sch.read(text, None, regs)
    it.generate(st, 0)
    tail = [dict(text="s_waitcnt lgkmcnt(0)", kind="wait", reads=set(), writes=set(), nops=1, lds=False, wait=0)]
    genb.check_stream(pro.ins + st.ins + tail, "as generated")
    waits = [n for n, i in enumerate(st.ins) if i["kind"] == "wait" and i["wait"] is not None and i["wait"] < 15]
    broken = st.ins[:waits[3]] + st.ins[waits[3] + 1:]
    with pytest.raises(SystemExit, match="in flight"):
        genb.check_stream(pro.ins + broken + tail, "a wait removed")


_spec_q = importlib.util.spec_from_file_location(
    "gen_dq_loop", os.path.join(ROOT, "chill-attention_amd", "csrc", "gen_dq_loop.py"))
genq = importlib.util.module_from_spec(_spec_q)
_spec_q.loader.exec_module(genq)


@pytest.mark.parametrize("elem", ["bf16", "f16"])
def test_dq_loop_generates_and_declares_what_it_writes(elem):
    """The generated, software-pipelined loop of the dQ kernel with register-resident Q and dO (csrc/gen_dq_loop.py):
    every path through the statement passes the hazard check, everything it writes is declared, all 256 accumulation
    registers are on its clobber list (the compiler must park nothing there), and a steady iteration holds what it
    is meant to."""
    c = genq.Config(elem)
    ins = genq.gen_statement(c)  # raises SystemExit if a hazard rule is broken
    outs, inputs, clob = genq.operand_lists(c)
    genq.check_clobbers(ins, outs, clob + genq.SPECIAL_CLOBBERS, c.name)
    assert {f"a{r}" for r in range(256)} <= set(clob)
    assert c.nvgpr + 32 + 2 + 16 + 4 <= 256   # its own registers, the two -delta blocks, LSE2, addresses, load offsets
    st = genq.Stream()
    genq.gen_body(c, st, 1, first=False)
    text = [i["text"] for i in st.ins]
    mf = [t for t in text if t.startswith("v_mfma")]
    assert len(mf) == 48
    # A_k and B_k take their B operands from the resident Q (a128 ..) and dO (a192 ..), C_(k-1) accumulates into a0 .. a127
    assert sum(", a[1" in t and t.split()[1].startswith("v[") for t in mf) >= 16
    acc = [t.split()[1].rstrip(",") for t in mf if t.split()[1].startswith("a[")]
    assert len(acc) == 16 and len(set(acc)) == 8
    # LDS: 8 transposed K operands of the tile before (two reads each), 8 V row chunks, 8 K row chunks of the next tile
    assert sum(t.startswith("ds_read_b64_tr_b16") for t in text) == 16 and sum(t.startswith("ds_read_b128") for t in text) == 16
    assert sum(t.startswith("v_exp_f32") for t in text) == 32 and sum(t.startswith("v_mul_f32") for t in text) == 32
    assert sum(t.startswith(c.cvt) for t in text) == 16 and text.count("s_barrier") == 1
    assert sum(t.startswith("global_load_lds_dwordx4") for t in text) == 4
    # the barrier stands behind the last MFMA that reads the tile before, and the loads of the tile three ahead behind it
    order = [n for n, t in enumerate(text) if t == "s_barrier" or t.startswith("global_load_lds") or "a[0:15], v[" in t or
             t.split()[1].startswith("a[")]
    bar = text.index("s_barrier")
    assert all(n < bar for n, t in enumerate(text) if t.startswith("v_mfma") and t.split()[1].startswith("a["))
    assert all(n > bar for n, t in enumerate(text) if t.startswith("global_load_lds"))
    assert order
