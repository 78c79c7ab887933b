"""Pins the CPU oracle (oracle/) before anything is compared against it.

Every check here is independent of the product: second statements of the same rule, brute force,
closed forms, special cases that reduce to library routines, finite differences.
"""

import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import MASK_INSTANCES, mask_id
from oracle import c_oracle as co
from oracle import chill_oracle as orc

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_predicate_two_statements_and_c_agree(m):
    name, args = m
    for n in (1, 10, 33, 500, 1030):
        pos = np.arange(n)
        a = orc.mask_pred(name, args, pos, pos)
        b = orc.mask_pred_flex(name, args, pos, pos)
        c = co.dense_mask(name, args, n)
        assert (a == b).all() and (a == c).all()


def test_predicate_special_cases():
    n = 257
    pos = np.arange(n)
    assert (orc.dense_mask("CausalChillMask", (), n) == np.tril(np.ones((n, n), bool))).all()
    assert (orc.dense_mask("SlidingWindowChillMask", (0, 0), n) == np.eye(n, dtype=bool)).all()
    assert orc.dense_mask("PrefixLMChillMask", (n,), n).all()
    assert orc.dense_mask("ChunkwiseChillMask", (n, 0), n).all()
    assert (orc.dense_mask("PrefixLMChillMask", (0,), n) == orc.dense_mask("CausalChillMask", (), n)).all()
    for back in (0, 3, 9):
        assert (orc.dense_mask("ChunkwiseChillMask", (1, back), n) == orc.dense_mask("SlidingWindowChillMask", (back, 0), n)).all()
    # banded: |q - k| structure
    sw = orc.dense_mask("SlidingWindowChillMask", (5, 2), n)
    d = pos[:, None] - pos[None, :]
    assert (sw == ((d <= 5) & (d >= -2))).all()


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_range_rules_equal_true_min_max(m):
    """The property ChillMask.verify checks (mask.py:737-761): analytic limits == enumerated."""
    name, args = m
    for n in (1, 10, 16, 500, 1030):
        dense = orc.dense_mask(name, args, n)
        for which, d in ((0, dense), (1, dense.T)):
            true = co.true_limits(name, args, which, n)
            rows = np.nonzero(d.any(axis=1))[0]
            # numpy restatement of the true limits, then both oracles' rules against them
            lo = d.argmax(axis=1)
            hi = n - 1 - d[:, ::-1].argmax(axis=1)
            assert (true[rows, 0] == lo[rows]).all() and (true[rows, 1] == hi[rows]).all()
            rule_c = co.rule_limits(name, args, which, n, n)
            fn = orc.k_range_for_q if which == 0 else orc.q_range_for_k
            rule_py = np.array([fn(name, args, i, n) for i in range(n)])
            assert (rule_c == rule_py).all()
            assert (rule_py[rows] == true[rows]).all()


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_full_ranges_sound_and_k_full_maximal(m):
    name, args = m
    for n in (10, 500, 1030):
        dense = orc.dense_mask(name, args, n)
        for tile in (16, 32, 64, 128):
            for b in range(0, n, tile):
                e = min(b + tile, n)
                lo, hi = orc.k_full_range_for_q(name, args, b, tile, n)
                hi_c = min(hi, n)
                if hi_c > lo:
                    assert dense[b:e, lo:hi_c].all()
                    if b + tile <= n:  # maximal: the neighbours are not visible to the whole tile
                        assert lo == 0 or not dense[b:e, lo - 1].all()
                        assert hi_c == n or not dense[b:e, hi_c].all()
                lo, hi = orc.q_full_range_for_k(name, args, b, tile, n)
                hi_c = min(hi, n)
                if hi_c > lo:
                    assert dense[lo:hi_c, b:e].all()


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_full_blocks_homogeneous(m):
    """mask.py:763-779: a block flagged full is all-True or all-False."""
    name, args = m
    n = 600
    dense = orc.dense_mask(name, args, n)
    for tq in (16, 32, 64, 128, 256):
        for tk in (16, 32, 64, 128, 256):
            h_py = orc.has_full_blocks(name, args, tq, tk, n)
            a = list(args) + [0, 0]
            assert bool(co.lib().oracle_has_full_blocks(co.MASK_IDS[name], a[0], a[1], tq, tk, n)) == bool(h_py)
            if not h_py:
                continue
            for q in range(0, n, tq):
                for k in range(0, n, tk):
                    f = orc.is_full_block(name, args, q, k, tq, tk, n)
                    assert bool(co.lib().oracle_is_full_block(co.MASK_IDS[name], a[0], a[1], q, k, tq, tk)) == bool(f)
                    if f:
                        t = dense[q : q + tq, k : k + tk]
                        assert t.all() or not t.any()


@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
@pytest.mark.parametrize("qrows", [True, False], ids=["qrows", "krows"])
def test_tile_decisions_python_c_and_bruteforce(m, qrows):
    name, args = m
    for T, seq_len in ((10, 10), (500, 500), (1030, 1030), (1030, 517), (512, 1)):
        for tin, tout in ((16, 16), (32, 64), (64, 32), (128, 128), (256, 64)):
            r_py = orc.tile_ranges(name, args, qrows, T, seq_len, tin, tout)
            r_c = co.tile_ranges(name, args, qrows, T, seq_len, tin, tout)
            assert (r_py == r_c).all(), (T, seq_len, tin, tout)
            assert co.check_tile_ranges(name, args, qrows, T, seq_len, tin, tout, r_c) == 0
            r_w = co.tile_ranges(name, args, qrows, T, seq_len, tin, tout, widened_q_full=True)
            assert co.check_tile_ranges(name, args, qrows, T, seq_len, tin, tout, r_w) == 0
            assert (r_w[:, :2] == r_c[:, :2]).all()


def test_tile_range_checker_catches_mistakes():
    """The brute-force checker itself must reject a dropped tile, a loose hull and an unsound full range."""
    name, args, T = "CausalChillMask", (), 512
    r = co.tile_ranges(name, args, True, T, T, 64, 64)
    assert co.check_tile_ranges(name, args, True, T, T, 64, 64, r) == 0
    bad = r.copy(); bad[3, 1] -= 1
    assert co.check_tile_ranges(name, args, True, T, T, 64, 64, bad) // 1000000 == 1
    bad = r.copy(); bad[3, 1] += 1
    assert co.check_tile_ranges(name, args, True, T, T, 64, 64, bad) // 1000000 == 2
    bad = r.copy(); bad[3, 3] += 1
    assert co.check_tile_ranges(name, args, True, T, T, 64, 64, bad) // 1000000 == 3


def test_widened_q_full_ranges_match_bruteforce_interval():
    """The q_full_range_for_k rules the HIP library adds for SW / Chunkwise / PrefixLM equal the
    exact brute-force interval whenever the key tile lies inside the sequence."""
    for name, args in (("SlidingWindowChillMask", (10, 4)), ("SlidingWindowChillMask", (128, 128)),
                       ("ChunkwiseChillMask", (10, 4)), ("ChunkwiseChillMask", (128, 2)), ("ChunkwiseChillMask", (77, 5)),
                       ("PrefixLMChillMask", (10,)), ("PrefixLMChillMask", (77,))):
        n = 700
        for tile in (16, 32, 64, 128):
            got = co.tile_ranges(name, args, False, n, n, tile, 1, widened_q_full=True)
            for t in range(n // tile):
                exact = orc.q_full_range_exact(name, args, t * tile, tile, n)
                assert exact is not None
                lo, hi = exact
                if got[t, 2] < got[t, 3]:
                    assert (got[t, 2], got[t, 3]) == (lo, hi), (name, args, tile, t)
                else:
                    assert hi <= lo or not orc.has_full_blocks(name, args, 1, tile, n)


def test_nnz_closed_forms_and_golden():
    for name, args in MASK_INSTANCES:
        for n in (1, 10, 500, 1030):
            assert orc.nnz(name, args, n) == int(orc.dense_mask(name, args, n).sum()) == co.nnz_bruteforce(name, args, n)
    with open(os.path.join(GOLDEN, "baseline_configs.json")) as f:
        golden = json.load(f)
    for c in golden["configs"]:
        assert orc.nnz(c["mask"], tuple(c["args"]), c["T"]) == c["nnz_per_head"], c["name"]
        fl = orc.flops(c["mask"], tuple(c["args"]), c["B"], c["H"], c["T"], c["D"], "fwd")
        assert abs(fl / 1e9 - c["fwd_gflop"]) <= 0.05 * max(1.0, c["fwd_gflop"] * 0.001) + 0.06, c["name"]


# ------------------------------------------------------------------------------- attention
def _rand(B, H, Hkv, T, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, T, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, Hkv, T, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, Hkv, T, D, generator=g, dtype=torch.float64)
    do = torch.randn(B, H, T, D, generator=g, dtype=torch.float64)
    return q, k, v, do


@pytest.mark.parametrize("m", MASK_INSTANCES[:5], ids=mask_id)
def test_reference_naive_equals_textbook_f64(m):
    name, args = m
    q, k, v, do = _rand(2, 4, 2, 45, 16)
    lens = torch.tensor([45, 17], dtype=torch.int32)
    for ln in (None, lens):
        qq, kk, vv = (x.clone().requires_grad_() for x in (q, k, v))
        out, rm = orc.reference_naive(name, args, qq, kk, vv, ln)
        dd = do * rm
        out.backward(dd)
        ref = orc.attention_f64(name, args, q.numpy(), k.numpy(), v.numpy(), dd.numpy(), None if ln is None else ln.numpy())
        o = ref["o"] * (1 if ln is None else rm.numpy())
        np.testing.assert_allclose(out.detach().numpy(), o, atol=1e-12, rtol=1e-10)
        np.testing.assert_allclose(qq.grad.numpy(), ref["dq"], atol=1e-11, rtol=1e-9)
        np.testing.assert_allclose(kk.grad.numpy(), ref["dk"], atol=1e-11, rtol=1e-9)
        np.testing.assert_allclose(vv.grad.numpy(), ref["dv"], atol=1e-11, rtol=1e-9)


def test_reference_naive_library_special_cases():
    q, k, v, _ = _rand(2, 3, 3, 64, 32, seed=3)
    full, _ = orc.reference_naive("FullChillMask", (), q, k, v)
    np.testing.assert_allclose(full.numpy(), F.scaled_dot_product_attention(q, k, v).numpy(), atol=1e-12)
    causal, _ = orc.reference_naive("CausalChillMask", (), q, k, v)
    np.testing.assert_allclose(causal.numpy(), F.scaled_dot_product_attention(q, k, v, is_causal=True).numpy(), atol=1e-12)
    diag, _ = orc.reference_naive("SlidingWindowChillMask", (0, 0), q, k, v)
    np.testing.assert_allclose(diag.numpy(), v.numpy(), atol=1e-12)  # every row sees only itself
    big, _ = orc.reference_naive("PrefixLMChillMask", (64,), q, k, v)
    np.testing.assert_allclose(big.numpy(), full.numpy(), atol=1e-12)


def test_attention_f64_gradients_by_finite_differences():
    name, args = "ChunkwiseChillMask", (3, 1)
    q, k, v, do = (x.numpy() for x in _rand(1, 2, 1, 7, 4, seed=5))
    base = orc.attention_f64(name, args, q, k, v, do, sm_scale=0.37)

    def loss(qq, kk, vv):
        return float((orc.attention_f64(name, args, qq, kk, vv, sm_scale=0.37)["o"] * do).sum())

    eps = 1e-6
    rng = np.random.default_rng(0)
    for key, arr, slot in (("dq", q, 0), ("dk", k, 1), ("dv", v, 2)):
        for _ in range(12):
            idx = tuple(rng.integers(0, s) for s in arr.shape)
            plus, minus = [q.copy(), k.copy(), v.copy()], [q.copy(), k.copy(), v.copy()]
            plus[slot][idx] += eps
            minus[slot][idx] -= eps
            fd = (loss(*plus) - loss(*minus)) / (2 * eps)
            assert abs(fd - base[key][idx]) < 1e-6, (key, idx, fd, base[key][idx])


def test_attention_invariants():
    name, args = "SlidingWindowChillMask", (4, 2)
    q, k, v, do = (x.numpy() for x in _rand(2, 2, 2, 33, 8, seed=7))
    r = orc.attention_f64(name, args, q, k, v, do)
    # rows are convex combinations of value rows
    assert (r["o"] <= v.max(axis=2, keepdims=True) + 1e-12).all() and (r["o"] >= v.min(axis=2, keepdims=True) - 1e-12).all()
    # scale symmetry of the scores: sum dQ.Q == sum dK.K
    assert abs((r["dq"] * q).sum() - (r["dk"] * k).sum()) < 1e-9
    # LSE2: closed form via logsumexp of the masked scaled scores
    s = np.einsum("bhqd,bhkd->bhqk", q, k) * 8 ** -0.5
    s = np.where(orc.dense_mask(name, args, 33)[None, None], s, -np.inf)
    lse = torch.logsumexp(torch.from_numpy(s), -1).numpy() * math.log2(math.e)
    np.testing.assert_allclose(r["lse2"], lse, atol=1e-12)
    np.testing.assert_allclose(orc.delta(r["o"], do), r["delta"], atol=1e-12)
    # fully masked rows (lens) give zeros and -inf
    r2 = orc.attention_f64(name, args, q, k, v, do, lens=np.array([33, 5]))
    assert (r2["o"][1, :, 5:] == 0).all() and np.isneginf(r2["lse2"][1, :, 5:]).all()
    assert (r2["dq"][1, :, 5:] == 0).all() and (r2["dk"][1, :, 5:] == 0).all() and (r2["dv"][1, :, 5:] == 0).all()


def test_lse2_dense_equals_the_direct_sum():
    """lse2_dense (torch, any device) against log2 of the plain sum of 2^(scaled score) over the visible
    keys, written without a max (small scores), with GQA and lens; and against the numpy textbook."""
    name, args = "ChunkwiseChillMask", (5, 1)
    q, k, _, _ = _rand(2, 4, 2, 21, 8, seed=11)
    lens = torch.tensor([21, 9], dtype=torch.int32)
    got = orc.lse2_dense(name, args, q, k, lens).numpy()
    dense = orc.dense_mask(name, args, 21)
    want = np.full((2, 4, 21), -np.inf)
    for b in range(2):
        for h in range(4):
            for i in range(int(lens[b])):
                tot = 0.0
                for j in range(int(lens[b])):
                    if dense[i, j]:
                        tot += 2.0 ** (float(q[b, h, i].double() @ k[b, h // 2, j].double()) * 8 ** -0.5 * math.log2(math.e))
                want[b, h, i] = math.log2(tot)
    np.testing.assert_allclose(got, want, atol=1e-10)
    np.testing.assert_allclose(got, orc.lse2(name, args, q.numpy(), k.numpy(), lens=lens.numpy()), atol=1e-10)
