"""Mask algebra of the product on the CPU: the Python ChillMask classes, the compiled
``__host__ __device__`` functors behind the C ABI, and the oracle must agree bit for bit, and the
compiled tile decisions must survive exhaustive enumeration (the method of the reference's
``ChillMask.verify``, mask.py:700-803, and its ``test_masks_verify``, test_chill_attention.py:79-81)."""

import ctypes

import numpy as np
import pytest

import chill_attention as ca
from chill_attention import _lib
from conftest import MASK_INSTANCES, make_mask, mask_id
from oracle import c_oracle as co
from oracle import chill_oracle as orc

REFERENCE_TEST_MASKS = MASK_INSTANCES[:5]


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_verify_1024(m):
    make_mask(m).verify(1024)


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_verify_odd_sizes(m):
    for n in (1, 10, 16, 33, 500):
        make_mask(m).verify(n)


def test_verify_rejects_a_wrong_rule():
    class Broken(ca.CausalChillMask):
        @staticmethod
        def k_range_for_q(q, seq_len, args):
            return np.zeros_like(q), q + 1  # off by one

    with pytest.raises(AssertionError):
        Broken().verify(64)

    class BrokenFull(ca.SlidingWindowChillMask):
        @staticmethod
        def k_full_range_for_q(qb, TILE_Q, seq_len, args):
            return 0, seq_len

    with pytest.raises(AssertionError):
        BrokenFull(10, 4).verify(128)


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_make_mask_equals_oracle(m):
    mask = make_mask(m)
    for n in (1, 10, 500, 1025):
        got = mask.make_mask(n).cpu().numpy()
        assert got.dtype == np.bool_ and got.shape == (n, n)
        assert (got == orc.dense_mask(m[0], m[1], n)).all()
        assert mask.nnz(n) == orc.nnz(m[0], m[1], n)


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_rows_and_columns_are_their_ranges(m):
    """The kernels mask a partial block of a built-in mask by comparing positions with the row's
    (column's) range instead of evaluating the predicate (kRowIsRange in csrc/chill_mask.h).  That is
    only right if every row and column of the dense mask is exactly its range, without holes: checked
    against the oracle's dense mask with the compiled limits."""
    mask = make_mask(m)
    desc = mask.descriptor()
    for n in (1, 10, 33, 500, 1025):
        dense = orc.dense_mask(m[0], m[1], n)
        pos = np.arange(n)
        for which, rows in ((0, dense), (1, dense.T)):
            lim = np.zeros((n, 2), dtype=np.int32)
            assert _lib.lib.chill_mask_limits(ctypes.byref(desc), which, n, n, lim.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))) == 0
            lo = np.maximum(lim[:, 0], 0)[:, None]
            hi = np.minimum(lim[:, 1], n - 1)[:, None]
            assert ((pos[None, :] >= lo) & (pos[None, :] <= hi) == rows).all(), (m, n, which)


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_python_rules_equal_oracle(m):
    mask = make_mask(m)
    name, args = m
    n = 300
    for pos in (0, 1, 9, 10, 77, 128, 299):
        assert tuple(int(x) for x in mask.k_range_for_q(np.int64(pos), n, args)) == orc.k_range_for_q(name, args, pos, n)
        assert tuple(int(x) for x in mask.q_range_for_k(np.int64(pos), n, args)) == orc.q_range_for_k(name, args, pos, n)
    for tq in (16, 32, 64, 128, 256):
        for b in range(0, n, tq):
            assert tuple(int(x) for x in mask.k_full_range_for_q(b, tq, n, args)) == orc.k_full_range_for_q(name, args, b, tq, n)
        for tk in (16, 32, 64, 128, 256):
            assert bool(mask.has_full_blocks(tq, tk, n, args)) == bool(orc.has_full_blocks(name, args, tq, tk, n))
            desc = mask.descriptor()
            assert bool(_lib.lib.chill_mask_has_full_blocks(ctypes.byref(desc), tq, tk, n)) == bool(mask.has_full_blocks(tq, tk, n, args))
            for q in range(0, n, tq):
                for k in range(0, n, tk):
                    py = bool(mask.is_full_block(q, k, tq, tk, n, args))
                    assert py == bool(orc.is_full_block(name, args, q, k, tq, tk, n))
                    assert py == bool(_lib.lib.chill_mask_is_full_block(ctypes.byref(desc), q, k, tq, tk, n))
    # Full and Causal: the reference defines q_full_range_for_k, it must match
    if name in ("FullChillMask", "CausalChillMask"):
        for b in range(0, n, 32):
            assert tuple(int(x) for x in mask.q_full_range_for_k(b, 32, n, args)) == orc.q_full_range_for_k(name, args, b, 32, n)


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
@pytest.mark.parametrize("pass_id", [_lib.PASS_FWD, _lib.PASS_DQ, _lib.PASS_DKDV], ids=["fwd", "dq", "dkdv"])
def test_compiled_tile_decisions(m, pass_id):
    """Tile ranges computed by the compiled functors: equal to the oracle's restatement of the
    reference logic where the reference defines the rule, and exhaustively sound everywhere."""
    mask = make_mask(m)
    name, args = m
    qrows = pass_id != _lib.PASS_DKDV
    for T, seq_len in ((10, 10), (500, 500), (1030, 1030), (1030, 517), (512, 1), (300, 299)):
        for tin, tout in ((16, 16), (32, 64), (32, 32), (64, 32), (128, 64), (256, 64), (128, 128)):
            got = mask._calc_tile_ranges(T, tin, tout, pass_id, seq_len).numpy().astype(np.int64)
            assert co.check_tile_ranges(name, args, qrows, T, seq_len, tin, tout, got) == 0
            want = co.tile_ranges(name, args, qrows, T, seq_len, tin, tout, widened_q_full=True)
            assert (got == want).all(), (T, seq_len, tin, tout)
            ref = orc.tile_ranges(name, args, qrows, T, seq_len, tin, tout)
            assert (got[:, :2] == ref[:, :2]).all()
            if qrows or name in ("FullChillMask", "CausalChillMask"):
                assert (got == ref).all()


@pytest.mark.parametrize("cfg", ["C2", "C3", "C4", "C5a"])
def test_compiled_tile_decisions_at_baseline_sizes(cfg):
    """Exhaustive enumeration at the full BASELINE sequence lengths, with the tile shapes the
    library actually uses (workgroup level and wave level)."""
    import json, os
    import torch

    with open(os.path.join(os.path.dirname(__file__), "golden", "baseline_configs.json")) as f:
        c = {x["name"]: x for x in json.load(f)["configs"]}[cfg]
    m = (c["mask"], tuple(c["args"]))
    mask = make_mask(m)
    dtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[c["dtype"]]
    from chill_attention.tiles import tile_config

    for pass_id in (_lib.PASS_FWD, _lib.PASS_DQ, _lib.PASS_DKDV):
        t = tile_config(mask, c["D"], dtype, pass_id)
        qrows = pass_id != _lib.PASS_DKDV
        for tin in (t["rows"], 32):
            got = mask._calc_tile_ranges(c["T"], tin, t["streamed"], pass_id).numpy().astype(np.int64)
            assert co.check_tile_ranges(m[0], m[1], qrows, c["T"], c["T"], tin, t["streamed"], got) == 0


def test_descriptor_and_str():
    m = ca.SlidingWindowChillMask(10, 4)
    assert str(m) == "SlidingWindowChillMask(10, 4)" and m.name == "SlidingWindowChillMask" and m.constargs == (10, 4)
    d = m.descriptor()
    assert (d.id, d.nargs, d.args[0], d.args[1]) == (_lib.MASK_SLIDING_WINDOW, 2, 10, 4)
    assert str(ca.CausalChillMask()) == "CausalChillMask()"
    assert ca.PrefixLMChillMask(7).descriptor().id == _lib.MASK_PREFIX_LM
    with pytest.raises(AssertionError):
        ca.ChillMask.__init__(ca.CausalChillMask(), constargs=[1, 2])  # not a tuple
    with pytest.raises(AssertionError):
        ca.ChillMask.__init__(ca.CausalChillMask(), constargs=("a",))

    class Custom(ca.ChillMask):
        mask = staticmethod(lambda q, k, seq_len, args: None)
        q_range_for_k = staticmethod(lambda k, seq_len, args: (0, 0))
        k_range_for_q = staticmethod(lambda q, seq_len, args: (0, 0))

    with pytest.raises(NotImplementedError):
        Custom().descriptor()
    with pytest.raises(ValueError):
        ca.SlidingWindowChillMask(1.5, 2).descriptor()


def test_base_class_defaults():
    class Minimal(ca.ChillMask):
        mask = staticmethod(lambda q, k, seq_len, args: None)
        q_range_for_k = staticmethod(lambda k, seq_len, args: (0, 0))
        k_range_for_q = staticmethod(lambda q, seq_len, args: (0, 0))

    m = Minimal()
    assert m.k_full_range_for_q(0, 16, 10, ()) == (0, 0) and m.q_full_range_for_k(0, 16, 10, ()) == (0, 0)
    assert not m.has_k_full_range() and not m.has_q_full_range() and not m.is_guaranteed_safe()
    assert m.q_lims_continious() and m.k_lims_continious()
    assert not m.has_full_blocks(16, 16, 10, ()) and not m.is_full_block(0, 0, 16, 16, 10, ())
    assert m.make_flex_mask(16) is None


@pytest.mark.parametrize("m", REFERENCE_TEST_MASKS, ids=mask_id)
def test_flex_mask_consistent(m):
    """Counterpart of the reference's test_flex_mask_consistent (test_chill_attention.py:332-345)."""
    from torch.nn.attention.flex_attention import create_mask

    mask = make_mask(m)
    n = 256
    flex = mask.make_flex_mask(n)
    assert flex is not None
    dense = create_mask(flex.mask_mod, None, None, n, n, device=mask.make_mask(1).device)[0, 0]
    assert (dense.cpu() == mask.make_mask(n).cpu()).all()


def test_plot_draws_both_panels(tmp_path):
    """plot() (reference mask.py:536-698) returns a two-panel figure; full blocks and predicate-free
    ranges are drawn as patches."""
    import matplotlib

    matplotlib.use("Agg")
    m = ca.SlidingWindowChillMask(40, 8)
    fig = m.plot(96, draw_full_blocks=16, plot_block_types=True, TILE_Q=16, TILE_K=16)
    assert len(fig.axes) == 2
    assert all(len(ax.lines) == 2 for ax in fig.axes)
    assert len(fig.axes[0].patches) > 0 and len(fig.axes[0].patches) == len(fig.axes[1].patches)
    fig.savefig(tmp_path / "mask.png")
    assert (tmp_path / "mask.png").stat().st_size > 0
    full = m._calc_full_ranges(96, 16).numpy()
    dense = m.make_mask(96).cpu().numpy()
    for i, (lo, hi) in enumerate(full):
        if hi > lo:
            assert dense[16 * i : 16 * i + 16, lo:hi].all()
