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
