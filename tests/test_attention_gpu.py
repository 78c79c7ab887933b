"""GPU parity tests: the HIP path (through the public op, i.e. through the C ABI) against the oracle.

The matrix mirrors the reference's test_simple_chill_forward / test_simple_chill_backward
(test/test_chill_attention.py:84-329): five masks x three dtypes x lens {none, tricky, random} x
contiguous / non-contiguous inputs x head dims x batch sizes x GQA shapes x sequence lengths, with
the reference's own tolerances.  The oracle (dense mask -> torch SDPA on fp32-upcast inputs, autograd
for the gradients) runs on the same device tensors.
"""

import math
import zlib

import numpy as np
import pytest
import torch

import chill_attention as ca
from chill_attention import _lib
from chill_attention.tiles import tile_config
from conftest import MASK_INSTANCES, make_mask, mask_id
from oracle import chill_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"

# reference tolerances (atol, rtol): test_chill_attention.py:167-172 (outputs), :316-321 (gradients)
OUT_TOL = {torch.float32: (2e-6, 1e-4), torch.float16: (1e-2, 1e-3), torch.bfloat16: (5e-2, 1e-2)}
GRAD_TOL = {torch.float32: (5e-5, 1e-3), torch.float16: (5e-3, 1e-3), torch.bfloat16: (1e-1, 1e-2)}


# the bar of the benchmark definition (atol = rtol): enforced on top of the reference's where head dim >= 64
NORTH_STAR = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def stable_seed(*key):
    """Seed from the test's parameters: the same in every process (Python salts hash() of strings)."""
    return zlib.crc32(repr(key).encode())


def check_close(got, want, dtype, tol, D, what):
    """got vs. want (fp32 oracle, cast to dtype) within the reference's (atol, rtol) and, for head
    dims >= 64, within the benchmark's atol = rtol as well; prints the margins."""
    want = want.to(dtype)
    diff = (got.float() - want.float()).abs()
    rel = (diff / want.float().abs().clamp_min(1e-3)).max().item()
    print(f"    {what}: max abs err {diff.max().item():.3e}, max rel err (|want| >= 1e-3) {rel:.3e}", flush=True)
    torch.testing.assert_close(got, want, atol=tol[0], rtol=tol[1], msg=lambda m: f"{what}: {m}")
    if D >= 64:
        ns = NORTH_STAR[dtype]
        if dtype == torch.bfloat16 and not what.startswith("O"):
            # bf16 gradients: P and dS are rounded to bf16 before the gradient MFMAs (as the reference does,
            # chill_bwd_dkdv.py:405-476, chill_bwd_dq.py:329-332) and the sum over a GQA group of 4-8 heads is
            # rounded once more, so a few elements per million land a bf16 ulp of a value in [1, 4) (2^-7 ..
            # 2^-6) off: the benchmark bar must hold for all but 1e-3 of the elements (three elements for the
            # tiny tensors of the matrix), three times its atol for all (keys that many queries attend to, such as
            # attention sinks, sum hundreds of such roundings)
            outside = int((diff > ns + ns * want.float().abs()).sum().item())
            assert outside <= max(3, 1e-3 * diff.numel()), f"{what}: {outside} of {diff.numel()} elements outside the benchmark bar {ns}"
            torch.testing.assert_close(got, want, atol=3 * ns, rtol=ns, msg=lambda m: f"{what} (three times the benchmark atol): {m}")
        else:
            torch.testing.assert_close(got, want, atol=ns, rtol=ns, msg=lambda m: f"{what} (benchmark bar {ns}): {m}")


def make_lens(kind, B, T, rng):
    """test_chill_attention.py:38-58"""
    if kind == "none":
        return None
    if kind == "tricky":
        choices = [1, 2, 5, T + 1, T, max(T // 2, 1), max(T // 4, 1)]
        vals = rng.choice(choices, B)
    else:
        vals = rng.integers(1, T + 1, B)
    return torch.tensor(vals, dtype=torch.int32, device=DEV)


def make_qkv(shape, dtype, noncontiguous):
    t = torch.testing.make_tensor(shape, dtype=dtype, device=DEV, noncontiguous=noncontiguous, low=-0.1, high=0.1)
    t.normal_()
    return t


# (noncontiguous, head_dim, B, (H, H_kv)) combinations covering every value of the reference matrix
# Launches of up to 256 or 512 q-tiles of 32 rows take the forward that splits the keys of a q-tile over
# its waves; (87, (6, 3)) keeps the ordinary forward covered at the shortest lengths (it is left out at
# the others), the shapes with B = 1 cover the other one at the longer ones.
FWD_SHAPES = [(False, 16, 1, (1, 1)), (True, 128, 7, (6, 3)), (False, 128, 1, (6, 1)), (True, 16, 7, (8, 8)),
              (False, 64, 87, (6, 3))]
# (the backward kernels have such a pair too: (87, (6, 3)) keeps the ordinary dQ / dK,dV covered at the shortest lengths)
BWD_SHAPES = [(False, 16, 1, (1, 1)), (True, 128, 7, (8, 2)), (False, 128, 16, (6, 1)), (True, 16, 7, (8, 8)),
              (False, 128, 1, (8, 1)), (False, 64, 87, (6, 3))]


@pytest.mark.parametrize("T", [1, 10, 16, 500, 512], ids=lambda x: f"time-{x}")
@pytest.mark.parametrize("lens_kind", ["none", "tricky", "random"], ids=lambda x: f"lens-{x}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("m", MASK_INSTANCES[:5], ids=mask_id)
def test_forward_matrix(m, dtype, lens_kind, T):
    mask = make_mask(m)
    rng = np.random.default_rng(stable_seed(m, str(dtype), lens_kind, T))
    for noncontig, D, B, (H, Hkv) in FWD_SHAPES:
        if B == 87 and T > 16:
            continue
        print(f"fwd {mask} {dtype} lens={lens_kind} T={T} noncontig={noncontig} D={D} B={B} H={H}/{Hkv}", flush=True)
        q = make_qkv((B, H, T, D), dtype, noncontig)
        k = make_qkv((B, Hkv, T, D), dtype, noncontig)
        v = make_qkv((B, Hkv, T, D), dtype, noncontig)
        lens = make_lens(lens_kind, B, T, rng)
        ref, res_mask = orc.reference_naive(m[0], m[1], q.float(), k.float(), v.float(), lens)
        out = ca.chill_attention(q, k, v, mask=mask, lens=lens) * res_mask
        check_close(out, ref, dtype, OUT_TOL[dtype], D, f"O (lens {None if lens is None else lens.tolist()})")


@pytest.mark.parametrize("T", [1, 10, 16, 800, 1025], ids=lambda x: f"time-{x}")
@pytest.mark.parametrize("lens_kind", ["none", "tricky", "random"], ids=lambda x: f"lens-{x}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("m", MASK_INSTANCES[:5], ids=mask_id)
def test_backward_matrix(m, dtype, lens_kind, T):
    mask = make_mask(m)
    rng = np.random.default_rng(stable_seed(m, str(dtype), lens_kind, T, "b"))
    for noncontig, D, B, (H, Hkv) in BWD_SHAPES:
        if B == 87 and T > 16:
            continue
        if T >= 800 and B == 16:
            B = 3  # keeps the dense oracle of the longest cases small; B=16 is covered at short T
        print(f"bwd {mask} {dtype} lens={lens_kind} T={T} noncontig={noncontig} D={D} B={B} H={H}/{Hkv}", flush=True)
        q = make_qkv((B, H, T, D), dtype, noncontig).requires_grad_()
        k = make_qkv((B, Hkv, T, D), dtype, noncontig).requires_grad_()
        v = make_qkv((B, Hkv, T, D), dtype, noncontig).requires_grad_()
        lens = make_lens(lens_kind, B, T, rng)
        qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
        ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens)
        # dO is drawn in fp32 as in the reference's test and rounded to the dtype once: the kernel and
        # the oracle differentiate against the same values
        dout = make_qkv((B, H, T, D), torch.float32, noncontig)
        dout = (dout * res_mask.broadcast_to(dout.shape)).to(dtype)
        ref.backward(dout.float())
        out = ca.chill_attention(q, k, v, mask=mask, lens=lens)
        out.backward(dout)
        tag = f"(lens {None if lens is None else lens.tolist()})"
        check_close(out.detach() * res_mask, ref.detach(), dtype, OUT_TOL[dtype], D, f"O {tag}")
        for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
            assert torch.isfinite(got).all(), name
            check_close(got, want, dtype, GRAD_TOL[dtype], D, f"{name} {tag}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_small_launch_forward(m, dtype):
    """The forward of launches far too small for the chip (32 query rows per workgroup, keys split over
    its waves, partial softmax states merged at the end): every mask instance, ragged lengths, GQA,
    rows that see no key, LSE included, against the oracle; and the same rows through the ordinary
    forward (the same problem with enough batch entries) within rounding."""
    mask = make_mask(m)
    rng = np.random.default_rng(stable_seed(m, str(dtype), "small"))
    for T, D, (H, Hkv) in ((1000, 64, (4, 2)), (333, 128, (2, 1)), (1024, 32, (3, 3)), (77, 16, (2, 2))):
        B = 2
        q, k, v = (make_qkv((B, h, T, D), dtype, False) for h in (H, Hkv, Hkv))
        lens = torch.tensor([T, max(1, T // 3)], dtype=torch.int32, device=DEV)
        ref, res_mask = orc.reference_naive(m[0], m[1], q.float(), k.float(), v.float(), lens)
        out, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens, return_lse=True)
        check_close(out * res_mask, ref, dtype, OUT_TOL[dtype], D, f"O small launch T={T} D={D}")
        # the ordinary forward on the same rows: copies of the batch make the launch large
        rep = 40 if T > 100 else 200
        big, big_lse = ca.chill_attention(q.repeat(rep, 1, 1, 1), k.repeat(rep, 1, 1, 1), v.repeat(rep, 1, 1, 1),
                                          mask=mask, lens=lens.repeat(rep), return_lse=True)
        torch.testing.assert_close(out.float(), big[:B].float(), atol=OUT_TOL[dtype][0], rtol=OUT_TOL[dtype][1])
        finite = torch.isfinite(big_lse[:B])
        assert (torch.isfinite(lse) == finite).all()
        # (the ordinary forward of 16-bit inputs folds the scale into Q and rounds it once more, as the
        # reference's PRESCALE_QK does, chill_fwd.py:158-159: its scores carry that rounding)
        lse_atol = {torch.float32: 1e-4, torch.float16: 5e-3, torch.bfloat16: 3e-2}[dtype]
        torch.testing.assert_close(lse[finite], big_lse[:B][finite], atol=lse_atol, rtol=1e-4)
        assert (lse[~finite] == big_lse[:B][~finite]).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("m", MASK_INSTANCES, ids=mask_id)
def test_small_launch_backward(m, dtype):
    """dQ and dK/dV of launches far too small for the chip (32 rows per workgroup, the streamed axis split over
    its waves, partial gradients added up at the end): every mask instance, ragged lengths, GQA, against
    the oracle; and the same rows through the ordinary kernels (enough batch entries) within rounding."""
    mask = make_mask(m)
    for T, D, (H, Hkv) in ((1000, 64, (4, 2)), (333, 128, (2, 1)), (1024, 32, (3, 3)), (77, 16, (2, 2))):
        B = 2
        q, k, v = (make_qkv((B, h, T, D), dtype, False).requires_grad_() for h in (H, Hkv, Hkv))
        lens = torch.tensor([T, max(1, T // 3)], dtype=torch.int32, device=DEV)
        qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
        ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens)
        dout = (make_qkv((B, H, T, D), torch.float32, False) * res_mask.broadcast_to((B, H, T, D))).to(dtype)
        ref.backward(dout.float())
        ca.chill_attention(q, k, v, mask=mask, lens=lens).backward(dout)
        small = [x.grad.clone() for x in (q, k, v)]
        for name, got, want in zip(("dq", "dk", "dv"), small, (qf.grad, kf.grad, vf.grad)):
            assert torch.isfinite(got).all(), name
            check_close(got, want, dtype, GRAD_TOL[dtype], D, f"{name} small launch T={T} D={D}")
        # the ordinary kernels on the same rows: copies of the batch make the launch large
        rep = 40 if T > 100 else 200
        qb, kb, vb = (x.detach().repeat(rep, 1, 1, 1).requires_grad_() for x in (q, k, v))
        ca.chill_attention(qb, kb, vb, mask=mask, lens=lens.repeat(rep)).backward(dout.repeat(rep, 1, 1, 1))
        for name, a, b in zip(("dq", "dk", "dv"), small, (qb.grad, kb.grad, vb.grad)):
            torch.testing.assert_close(a.float(), b[:B].float(), atol=3 * GRAD_TOL[dtype][0], rtol=10 * GRAD_TOL[dtype][1],
                                       msg=lambda msg: f"{name} T={T} D={D}: {msg}")


# Small launches of more 32-row tiles than the chip has CUs: forward and dQ workgroups of eight waves take two tiles side
# by side (tile j from the end and tile j from the start of a head).  An even and an odd number of tiles per head (the
# middle one has no partner), GQA, lens that leave one of the two tiles, or both, behind the end of the sequence.
TWO_TILE_CASES = [
    ("prefix-lm-f32-D64", torch.float32, 1, 8, 8, 2048, 64, ("PrefixLMChillMask", (1024,)), None),
    ("causal-f32-D32-odd-lens", torch.float32, 3, 3, 3, 1500, 32, ("CausalChillMask", ()), (1500, 40, 777)),
    ("causal-bf16-D128-gqa-odd-lens", torch.bfloat16, 2, 6, 2, 1111, 128, ("CausalChillMask", ()), (1111, 1)),
    ("sliding-f16-D128-lens", torch.float16, 1, 5, 5, 2048, 128, ("SlidingWindowChillMask", (100, 7)), (1025,)),
    ("chunkwise-f32-D16", torch.float32, 2, 4, 4, 1990, 16, ("ChunkwiseChillMask", (100, 1)), None),
    ("full-f32-D64-gqa", torch.float32, 1, 12, 3, 1000, 64, ("FullChillMask", ()), (999,)),
    # fp32 takes these kernels far beyond that: 2048 tiles under a causal mask in all three passes
    ("causal-f32-D64-2048-tiles-lens", torch.float32, 2, 16, 16, 2048, 64, ("CausalChillMask", ()), (2048, 1500)),
    # rows of 512 bytes: two areas do not fit in LDS, one tile per workgroup, longest first across the heads
    ("prefix-lm-f32-D128-1536-tiles-gqa", torch.float32, 1, 24, 12, 2048, 128, ("PrefixLMChillMask", (300,)), None),
    # a few fp32 heads of a long sequence
    ("causal-f32-D64-T8192-gqa-lens", torch.float32, 1, 2, 1, 8192, 64, ("CausalChillMask", ()), (8000,)),
    ("full-f32-D128-T8200", torch.float32, 1, 2, 2, 8200, 128, ("FullChillMask", ()), None),
    # the same with 16-bit inputs: 512 tiles under a causal mask (at head dim 64 all three passes)
    ("causal-bf16-D64-T8192", torch.bfloat16, 1, 2, 2, 8192, 64, ("CausalChillMask", ()), None),
    ("prefix-lm-f16-D128-T16384-lens", torch.float16, 1, 1, 1, 16384, 128, ("PrefixLMChillMask", (5000,)), (16001,)),
]


@pytest.mark.parametrize("case", TWO_TILE_CASES, ids=lambda c: c[0])
def test_small_launch_with_two_tiles_per_workgroup(case):
    """Forward (O and LSE2, chill_fwd.py:215-330) and backward (chill_bwd_dq.py:300-394, chill_bwd_dkdv.py:347-508) of
    small launches whose forward and dQ workgroups hold two tiles (asserted from the tile report: 32 rows per tile,
    twice the LDS of one tile), against the oracle."""
    _, dtype, B, H, Hkv, T, D, m, lens = case
    mask = make_mask(m)
    for pass_id, heads, tiles in ((_lib.PASS_FWD, H, 2), (_lib.PASS_DQ, H, 2), (_lib.PASS_DKDV, Hkv, 1)):
        cfg = tile_config(mask, D, dtype, pass_id, seq_len=T, batch_heads=B * heads)
        if cfg["rows"] != 32:
            # (only the forward of every case is meant to take the small kernel: at head dim 128 the 16-bit backward of
            # these sizes takes ordinary kernels)
            assert pass_id != _lib.PASS_FWD and (dtype != torch.float32 or pass_id == _lib.PASS_DKDV), f"pass {pass_id} served by {cfg}"
            continue
        single = tile_config(mask, D, dtype, pass_id, seq_len=32, batch_heads=1)
        assert (cfg["waves"], cfg["streamed"]) == (4, 32) and single["rows"] == 32
        if 2 * single["lds_bytes"] > 160 * 1024:
            tiles = 1
        assert cfg["lds_bytes"] == tiles * single["lds_bytes"], f"pass {pass_id}: {cfg} against {single}"
    torch.manual_seed(stable_seed(case[0]))
    q, k, v = (make_qkv((B, h, T, D), dtype, False).requires_grad_() for h in (H, Hkv, Hkv))
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    dout = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    out, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens_t, return_lse=True)
    out.backward(dout)
    qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
    ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens_t)
    ref.backward(dout.float() * res_mask)
    check_close(out.detach() * res_mask, ref.detach(), dtype, OUT_TOL[dtype], D, "O")
    want_lse = orc.lse2_dense(m[0], m[1], q.detach(), k.detach(), lens_t)
    seen = torch.isfinite(want_lse)
    torch.testing.assert_close(lse[seen].double(), want_lse[seen], atol=1e-4 if dtype == torch.float32 else 2e-2, rtol=1e-4)
    assert (lse[~seen] == (-math.inf if lens is None else lse[~seen])).all()
    for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
        assert torch.isfinite(got).all(), name
        check_close(got, want, dtype, GRAD_TOL[dtype], D, name)
    if lens is not None:
        for b, n in enumerate(lens):
            assert (out[b, :, n:] == 0).all() and (q.grad[b, :, n:] == 0).all() and (k.grad[b, :, n:] == 0).all()


@pytest.mark.parametrize("D", [32, 64, 128])
def test_fp32_beyond_the_small_launch_kernels(D):
    """The ordinary fp32 kernels (a wave owns 32 rows and walks all their blocks), which fp32 launches leave to the
    small-launch kernels up to thousands of 32-row tiles: grids beyond those limits (route asserted), against the oracle;
    GQA, lens, a ragged end."""
    for m, T, B, H, Hkv, lens in ((("CausalChillMask", ()), 4100, 8, 16, 8, (4100, 3000, 77, 4099, 1, 4100, 2222, 4000)),
                                  (("SlidingWindowChillMask", (300, 20)), 2100, 2, 12, 6, (2100, 1000)),
                                  (("PrefixLMChillMask", (1000,)), 4100, 8, 16, 16, None)):
        lens = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
        mask = make_mask(m)
        for pass_id, heads in ((_lib.PASS_FWD, H), (_lib.PASS_DQ, H), (_lib.PASS_DKDV, Hkv)):
            cfg = tile_config(mask, D, torch.float32, pass_id, seq_len=T, batch_heads=B * heads)
            assert cfg["rows"] == 128, f"pass {pass_id} served by {cfg}"
        torch.manual_seed(stable_seed(m, D, "fp32 long"))
        q, k, v = (make_qkv((B, h, T, D), torch.float32, False).requires_grad_() for h in (H, Hkv, Hkv))
        dout = torch.randn(B, H, T, D, device=DEV)
        out = ca.chill_attention(q, k, v, mask=mask, lens=lens)
        out.backward(dout)
        qf, kf, vf = (x.detach().clone().requires_grad_() for x in (q, k, v))
        ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens)
        ref.backward(dout * res_mask)
        check_close(out.detach() * res_mask, ref.detach(), torch.float32, OUT_TOL[torch.float32], D, f"O {m[0]}")
        for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
            check_close(got, want, torch.float32, GRAD_TOL[torch.float32], D, f"{name} {m[0]}")


def test_cpp_operator_matches_python_operator():
    """Eager calls go through the operator registered from C++; the torch.library operators (what
    torch.compile sees) must give the same bits, forward and backward, on the same kernels."""
    assert _lib.torch_operator() is not None, "libchill_attention_torch.so has not been built"
    mask = ca.SlidingWindowChillMask(100, 20)
    B, H, Hkv, T, D = 3, 4, 2, 700, 64
    q = make_qkv((B, H, T, D), torch.bfloat16, True).requires_grad_()
    k = make_qkv((B, Hkv, T, D), torch.bfloat16, True).requires_grad_()
    v = make_qkv((B, Hkv, T, D), torch.bfloat16, False).requires_grad_()
    lens = torch.tensor([T, 1, 333], dtype=torch.int32, device=DEV)
    do = make_qkv((B, H, T, D), torch.bfloat16, False)
    out, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens, return_lse=True)
    out.backward(do)
    got = [out.detach(), lse.detach()] + [x.grad.clone() for x in (q, k, v)]
    for x in (q, k, v):
        x.grad = None
    from chill_attention import chill as chill_mod

    out2, lse2 = chill_mod._chill_attention(q, k, v, lens, mask.name, mask.constargs, D ** -0.5, True, False, "ieee", False)
    out2.backward(do)
    want = [out2.detach(), lse2.detach()] + [x.grad for x in (q, k, v)]
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    # no gradient asked for: no LSE is kept, the output is the same
    with torch.no_grad():
        quiet = ca.chill_attention(q, k, v, mask=mask, lens=lens)
        assert torch.equal(quiet, out2.detach()) and not quiet.requires_grad and quiet.grad_fn is None


@pytest.mark.parametrize("D", [32, 64, 256])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_other_head_dims(dtype, D):
    for m in (MASK_INSTANCES[1], MASK_INSTANCES[3]):
        mask = make_mask(m)
        B, H, Hkv, T = 2, 4, 2, 333
        q, k, v = (make_qkv((B, h, T, D), dtype, False).requires_grad_() for h in (H, Hkv, Hkv))
        qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
        ref, _ = orc.reference_naive(m[0], m[1], qf, kf, vf, None)
        dout = torch.randn_like(ref)
        ref.backward(dout)
        out = ca.chill_attention(q, k, v, mask=mask)
        out.backward(dout.to(dtype))
        check_close(out.detach(), ref.detach(), dtype, OUT_TOL[dtype], D, "O")
        for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
            check_close(got, want, dtype, GRAD_TOL[dtype], D, name)


@pytest.mark.parametrize("dtype,D,T", [(torch.bfloat16, 128, 700), (torch.float16, 64, 300), (torch.float32, 32, 130), (torch.bfloat16, 128, 2300)], ids=str)
def test_zero_scale_is_uniform_attention(dtype, D, T):
    """sm_scale = 0: every visible key weighs the same (chill_fwd.py:213-214 scales, then masks), dQ and dK
    vanish; a non-finite scale is refused."""
    m = MASK_INSTANCES[1]
    mask = make_mask(m)
    B, H = 2, 8
    q, k, v = (torch.randn(B, H, T, D, device=DEV, dtype=dtype).requires_grad_() for _ in range(3))
    do = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    out = ca.chill_attention(q, k, v, mask=mask, sm_scale=0.0)
    out.backward(do)
    vf = v.detach().float().clone().requires_grad_()
    want = torch.cumsum(vf, dim=2) / torch.arange(1, T + 1, device=DEV)[None, None, :, None]
    want.backward(do.float())
    assert torch.isfinite(out).all()
    check_close(out.detach(), want.detach(), dtype, OUT_TOL[dtype], D, "O")
    check_close(v.grad, vf.grad, dtype, GRAD_TOL[dtype], D, "dv")
    assert (q.grad == 0).all() and (k.grad == 0).all()
    with pytest.raises(ValueError):
        ca.chill_attention(q, k, v, mask=mask, sm_scale=float("inf"))


def test_cpu_tensor_next_to_gpu_tensors_is_refused():
    q = torch.randn(1, 2, 64, 64, device=DEV)
    with pytest.raises(ValueError):
        ca.chill_attention(q, q.cpu(), q, mask=ca.CausalChillMask())
    with pytest.raises(ValueError):
        ca.chill_attention(q, q, q, mask=ca.CausalChillMask(), lens=torch.tensor([5], dtype=torch.int32))


def test_lse_and_fully_masked_rows():
    """LSE2 is base 2 and includes the scale (chill_fwd.py:328); rows that see no key give O = 0 and
    LSE2 = -inf; rows at or beyond lens give O = 0."""
    m = ("SlidingWindowChillMask", (3, 0))
    mask = make_mask(m)
    B, H, T, D = 2, 2, 200, 64
    q, k, v = (torch.randn(B, H, T, D, device=DEV) for _ in range(3))
    lens = torch.tensor([200, 37], dtype=torch.int32, device=DEV)
    o, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens, sm_scale=0.2, return_lse=True)
    ref = orc.attention_f64(m[0], m[1], q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy(), lens=lens.cpu().numpy(), sm_scale=0.2)
    assert lse.shape == (B, H, T) and lse.dtype == torch.float32
    np.testing.assert_allclose(lse[0].cpu().numpy(), ref["lse2"][0], atol=2e-5, rtol=1e-5)
    np.testing.assert_allclose(lse[1, :, :37].cpu().numpy(), ref["lse2"][1, :, :37], atol=2e-5, rtol=1e-5)
    np.testing.assert_allclose(o.cpu().numpy(), ref["o"], atol=2e-5, rtol=1e-4)
    assert (o[1, :, 37:] == 0).all()
    # a mask under which late rows see nothing once lens cuts the keys: chunk 0 only is valid
    m2 = ("ChunkwiseChillMask", (16, 0))
    lens2 = torch.tensor([16, 200], dtype=torch.int32, device=DEV)
    o2, lse2 = ca.chill_attention(q, k, v, mask=make_mask(m2), lens=lens2, return_lse=True)
    assert (o2[0, :, 16:] == 0).all() and torch.isfinite(o2).all()
    # sm_scale default and custom agree with the closed form
    o3 = ca.chill_attention(q, k, v, mask=ca.FullChillMask(), sm_scale=D ** -0.5)
    o4 = ca.chill_attention(q, k, v, mask=ca.FullChillMask())
    assert torch.equal(o3, o4)


# Forward kernels by the route a launch takes: (rows, waves) that chill_tile_config_for_shape reports.
#   (256, 8): the generated loop of 16-bit inputs at head dim 128 (fwd_fast_q_tiles; a q-tile whose sums leave the
#             range of the reference-free softmax is voted on and computed again by fwd_q_tile on the same LDS ring)
#   (128, 4): head dim 64, 16-bit: the generated loop of that shape, same vote; head dim 128 at T <= 1024, head dim 32,
#             fp32: fwd_q_tile itself (16-bit: the guarded raise of the reference; fp32: the running max); head dim 256,
#             16-bit: fwd_regs_kernel
#   (32, 4):  fwd_small_kernel
# drift: which query rows carry the direction the scores grow along ("all"; "low": the lower half of the sequence, which
# in a paired launch is the SECOND q-tile of every pair; "high": the upper half, the first q-tile of every pair; "wave":
# the 32 rows 160 .. 191 of every fourth block of 256 rows).
RAMP_CASES = [
    # id, dtype, D, B, H, H_kv, T, (rows, waves), masks, drift, lens
    ("d128-loop-unpaired", torch.bfloat16, 128, 2, 8, 8, 2048, (256, 8), (0, 1), "all", None),
    ("d128-loop-unpaired-f16", torch.float16, 128, 2, 8, 2, 2048, (256, 8), (0, 1), "all", None),
    ("d128-loop-paired", torch.bfloat16, 128, 4, 16, 16, 2048, (256, 8), (1, 7), "all", None),
    ("d128-loop-paired-f16", torch.float16, 128, 4, 16, 4, 2048, (256, 8), (0, 1), "all", None),
    ("d128-loop-paired-second-only", torch.bfloat16, 128, 4, 16, 16, 2048, (256, 8), (0, 1, 7), "low", None),
    ("d128-loop-paired-first-only", torch.float16, 128, 4, 16, 16, 2048, (256, 8), (0, 1), "high", None),
    ("d128-loop-paired-one-wave", torch.bfloat16, 128, 4, 16, 16, 2048, (256, 8), (0, 1, 7), "wave", None),
    ("d128-loop-paired-lens", torch.bfloat16, 128, 4, 16, 8, 2048, (256, 8), (0, 1, 7), "all", (2048, 1500, 300, 2047)),
    ("d128-loop-paired-lens-f16", torch.float16, 128, 4, 16, 16, 2048, (256, 8), (1,), "low", (700, 2048, 1, 1025)),
    # "step": the scores jump by the whole growth at key T / 2 instead of climbing to it: more than a sum inside the
    # loop can take within one tile, so these q-tiles are voted on and computed again by fwd_q_tile on the same LDS ring
    ("d128-loop-paired-step", torch.bfloat16, 128, 4, 16, 16, 2048, (256, 8), (0, 1, 7), "step", None),
    ("d128-loop-paired-step-f16", torch.float16, 128, 4, 16, 8, 2048, (256, 8), (0, 1), "step-low", (2048, 1500, 300, 2047)),
    ("d128-loop-unpaired-step", torch.bfloat16, 128, 2, 8, 8, 2048, (256, 8), (0, 1), "step-wave", None),
    ("d64-loop-step", torch.bfloat16, 64, 8, 16, 16, 2048, (128, 4), (0, 1, 7), "step-low", None),
    ("d64-loop-step-f16", torch.float16, 64, 3, 8, 4, 1024, (128, 4), (0, 1), "step", None),
    ("d64-loop", torch.bfloat16, 64, 3, 8, 8, 1024, (128, 4), (0, 1, 4), "all", None),
    ("d64-loop-f16", torch.float16, 64, 3, 8, 4, 1024, (128, 4), (0, 1, 4), "all", None),
    ("d64-loop-paired-second-only", torch.float16, 64, 8, 16, 16, 2048, (128, 4), (0, 1, 7), "low", None),
    ("d64-loop-paired-lens", torch.bfloat16, 64, 8, 16, 16, 2048, (128, 4), (1, 7), "wave", (2048, 3, 999, 1024, 2048, 1500, 64, 129)),
    ("d128-short-row", torch.bfloat16, 128, 8, 8, 8, 768, (128, 4), (0, 1), "all", None),
    ("d128-short-row-f16", torch.float16, 128, 8, 8, 8, 1024, (128, 4), (1, 4), "wave", None),
    ("d32", torch.float16, 32, 3, 8, 8, 1024, (128, 4), (0, 1), "all", None),
    ("d32-bf16", torch.bfloat16, 32, 3, 8, 8, 1024, (128, 4), (0, 1), "all", None),
    ("d256-regs", torch.bfloat16, 256, 2, 8, 8, 2048, (128, 4), (0, 1), "all", None),
    ("d256-regs-f16", torch.float16, 256, 2, 8, 8, 2048, (128, 4), (0, 1, 7), "wave", None),
    # (fp32: more than 2048 tiles of 32 rows, where the small-launch kernels stop)
    ("f32-d64", torch.float32, 64, 8, 10, 10, 1024, (128, 4), (0, 1), "all", None),
    ("f32-d128", torch.float32, 128, 8, 10, 10, 1024, (128, 4), (0, 1), "all", None),
    ("small-d64", torch.bfloat16, 64, 1, 2, 2, 1024, (32, 4), (0, 1), "all", None),
    ("small-d128-f16", torch.float16, 128, 1, 2, 2, 1024, (32, 4), (0, 1), "all", None),
    ("small-d256", torch.bfloat16, 256, 1, 2, 2, 1024, (32, 4), (0, 1), "all", None),
]
# what a row's scores have to rise by over its first keys (log2 units) before the reference-free softmax of the
# generated loops leaves its range (chill_fwd_fast.h: bf16 l > 2^60; fp16 one block sum > 2^15, which a row sum above
# 2^21 implies for up to 64 blocks), and what the test feeds
RAMP_TRIP = {torch.bfloat16: 60.0, torch.float16: 21.0, torch.float32: 0.0}
RAMP_GROWTH = {torch.bfloat16: 400.0, torch.float16: 60.0, torch.float32: 60.0}
STEP_GROWTH = {torch.bfloat16: 400.0, torch.float16: 300.0}


@pytest.mark.parametrize("case", RAMP_CASES, ids=lambda c: c[0])
def test_reference_max_is_raised_along_the_keys(case):
    """Scores that grow by RAMP_GROWTH (log2 units) along the key axis, for the rows selected by `drift`: the
    forward's reference max has to follow them.  Every forward kernel has its own way (running max; a guarded raise;
    the softmax of the generated loops, which raises a row's reference only when a sum leaves a guarded range, in an
    out-of-line block of the generated statement and in the steps around it): one case per kernel and way, with the
    route asserted from the tile table.  O and LSE2 against the
    oracle (chill_fwd.py:188-286 is the running-max softmax all of them must equal)."""
    _, dtype, D, B, H, Hkv, T, route, mask_ix, drift, lens = case
    step = drift.startswith("step")
    drift = {"step": "all", "step-low": "low", "step-wave": "wave"}.get(drift, drift)
    growth = STEP_GROWTH[dtype] if step else RAMP_GROWTH[dtype]
    torch.manual_seed(7)
    q = torch.randn(B, H, T, D, device=DEV) * 0.5
    k = torch.randn(B, Hkv, T, D, device=DEV) * 0.5
    v = torch.randn(B, Hkv, T, D, device=DEV)
    # a common direction whose weight in k grows with the key position: score(q, k_t) ~ t * growth / T (log2 units)
    # for the rows that carry it; the other rows have no component along it at all
    u = torch.nn.functional.normalize(torch.randn(D, device=DEV), dim=0)
    rows = torch.arange(T, device=DEV)
    carries = {"all": rows >= 0, "low": rows < T // 2, "high": rows >= T // 2,
               "wave": ((rows // 256) % 4 == 3) & ((rows % 256) // 32 == 5)}[drift]
    q = q - (q @ u)[..., None] * u
    q = q + 4.0 * carries[None, None, :, None] * u
    ramp = torch.arange(T, device=DEV, dtype=torch.float32) / T
    if step:
        ramp = (ramp >= (0.25 if drift == "low" else 0.5)).float()
    k = k + (growth * (D ** 0.5) / (4.0 * 1.4427)) * ramp[None, None, :, None] * u
    q, k, v = (x.to(dtype) for x in (q, k, v))
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    for m in (MASK_INSTANCES[i] for i in mask_ix):
        mask = make_mask(m)
        cfg = tile_config(mask, D, dtype, _lib.PASS_FWD, seq_len=T, batch_heads=B * H)
        assert (cfg["rows"], cfg["waves"]) == route, f"{m}: this shape is served by {cfg}, the case is meant for {route}"
        print(f"ramp {case[0]} {mask}: {cfg}", flush=True)
        ref, res_mask = orc.reference_naive(m[0], m[1], q.float(), k.float(), v.float(), lens_t)
        want_lse = orc.lse2_dense(m[0], m[1], q, k, lens_t)
        if RAMP_TRIP[dtype] > 0:
            # the inputs do what the case is for: in rows that carry the direction the exponent rises by more than the
            # reference-free softmax can hold above ANY reference taken from a row's first 64 keys (every mask here
            # starts its rows at key 0; LSE2 >= the largest exponent; the exponent of the first keys is below
            # growth * 64 / T plus the noise of the other directions, a fraction of a unit)
            risen = want_lse - growth * 64.0 / T - 4.0 > RAMP_TRIP[dtype]
            hit = risen & carries[None, None, :]
            assert hit.any(), "no row leaves the range"
            if drift != "all":
                quiet = want_lse[:, :, ~carries]
                quiet = quiet[torch.isfinite(quiet)]
                assert quiet.max() < 14.0 and quiet.min() > -6.0, "rows without the direction must stay inside the range"
        out, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens_t, return_lse=True)
        atol, rtol = OUT_TOL[dtype]
        if dtype == torch.float32:
            # raw scores reach several hundred here: their fp32 rounding alone moves P by ~3e-5 relative, whatever
            # the order of the sums, so the fp32 bar of the other tests (2e-6 / 1e-4) is out of reach for both sides
            atol, rtol = 1e-5, 1e-3
        assert torch.isfinite(out).all()
        torch.testing.assert_close(out * res_mask, ref.to(dtype), atol=atol, rtol=rtol)
        # LSE2 (up to `growth` in size): rows inside lens that see a key; the rest is 0 or -inf by definition
        seen = torch.isfinite(want_lse)
        assert torch.isfinite(lse[seen]).all()
        tight = 1e-2 if dtype != torch.float32 else 1e-3
        err = (lse.double() - want_lse).abs()
        if dtype != torch.float32 and D in (64, 128) and route != (32, 4) and not (D == 128 and route == (128, 4)):
            # The generated loops take Q already multiplied by scale * log2(e) and rounded to the input type (what the
            # reference's PRESCALE_QK does, chill_fwd.py:120-127, chill_bwd_dkdv.py:118): the exponent of a (query, key)
            # pair then carries the rounding errors of D products, each up to eps * |q_d * k_d| * scale * log2(e), in sum
            # at most eps * |q| * |k| * scale * log2(e).  (The keys of this test reach a norm of several hundred: the
            # bound is ~1.4 log2 units where LSE2 is ~400; the observed errors reach half of it.)
            eps = {torch.bfloat16: 2.0 ** -9, torch.float16: 2.0 ** -12}[dtype]
            k_norm = k.float().norm(dim=-1).amax(dim=-1)  # [B, H_kv]
            k_norm = k_norm.repeat_interleave(H // Hkv, dim=1)[..., None]
            loose = eps * (D ** -0.5 * 1.4427) * q.float().norm(dim=-1) * k_norm
            assert (err[seen] <= (tight + loose)[seen]).all(), (err - loose)[seen].max()
        else:
            assert (err[seen] <= tight + 1e-4 * want_lse[seen].abs()).all(), err[seen].max()


# dK/dV at 16-bit head dim 128 on long sequences and full grids: K in registers, runs of predicate-free tiles in the
# generated loop (chill_bwd_dkdv_regs.h, gen_bwd_loop.py).  id, dtype, B, H, H_kv, T, mask, lens
DKDV_REGS_CASES = [
    ("causal", torch.bfloat16, 2, 16, 16, 4096, ("CausalChillMask", ()), None),
    ("causal-gqa-lens-f16", torch.float16, 4, 16, 8, 4096, ("CausalChillMask", ()), (4096, 4000, 33, 2049)),
    ("full-gqa-ragged", torch.bfloat16, 2, 32, 16, 4100, ("FullChillMask", ()), None),
    ("full-lens-f16", torch.float16, 2, 16, 16, 4130, ("FullChillMask", ()), (4130, 3000)),
    ("prefix-lm", torch.bfloat16, 2, 16, 16, 4096, ("PrefixLMChillMask", (1024,)), None),
    ("prefix-lm-gqa-ragged", torch.float16, 1, 64, 32, 4111, ("PrefixLMChillMask", (77,)), (4001,)),
    # longer sequences (dQ takes its register-resident kernel, chill_bwd_dq_gen.h and gen_dq_loop.py, from 4097 keys on, under a
    # full mask from 2048, on grids of at least 512 workgroups)
    ("long-causal", torch.bfloat16, 1, 16, 16, 8192, ("CausalChillMask", ()), None),
    ("long-causal-gqa-lens-f16", torch.float16, 2, 16, 8, 8192, ("CausalChillMask", ()), (8192, 5000)),
    ("long-full-ragged", torch.bfloat16, 1, 32, 16, 8200, ("FullChillMask", ()), None),
    ("long-prefix-lm-ragged-lens-f16", torch.float16, 1, 32, 32, 8207, ("PrefixLMChillMask", (1024,)), (8100,)),
    # chunks of a multiple of a wave's 64 key rows: every block inside the band is predicate-free (dQ keeps its ordinary kernel);
    # runs that start in the middle of a workgroup's tiles and end before its last, a GQA group, a ragged end
    ("chunkwise-128x2-f16", torch.float16, 1, 16, 16, 8192, ("ChunkwiseChillMask", (128, 2)), None),
    ("chunkwise-64x4-gqa-lens", torch.bfloat16, 4, 16, 8, 4096, ("ChunkwiseChillMask", (64, 4)), (4096, 3000, 77, 4001)),
    ("chunkwise-1024x1-ragged-f16", torch.float16, 1, 32, 32, 4140, ("ChunkwiseChillMask", (1024, 1)), None),
    ("chunkwise-192x0", torch.bfloat16, 1, 32, 32, 4096, ("ChunkwiseChillMask", (192, 0)), None),
    # shorter sequences: from 1024 keys on under a full mask, from 3072 under causal-like masks
    ("full-T1024-gqa-lens", torch.bfloat16, 16, 16, 8, 1024, ("FullChillMask", ()), (1024, 1000, 5, 513, 1024, 1, 256, 257, 1023, 700, 64, 1024, 33, 900, 512, 1024)),
    ("full-T1100-ragged-f16", torch.float16, 8, 16, 16, 1100, ("FullChillMask", ()), None),
    ("causal-T3072", torch.bfloat16, 3, 16, 16, 3072, ("CausalChillMask", ()), None),
    # (one workgroup per CU under a full mask)
    ("full-256-workgroups-gqa-f16", torch.float16, 1, 32, 16, 4100, ("FullChillMask", ()), (4001,)),
    ("prefix-lm-T3300-gqa-ragged-lens-f16", torch.float16, 6, 16, 8, 3300, ("PrefixLMChillMask", (100,)), (3300, 3000, 3299, 77, 1700, 3300)),
    # sliding windows of 4096 keys and more: a long loop again, with masked tiles at both ends of a wave's run
    ("sliding-4096+0", torch.bfloat16, 2, 16, 16, 8192, ("SlidingWindowChillMask", (4096, 0)), None),
    ("sliding-3000+2000-gqa-ragged-lens-f16", torch.float16, 1, 32, 16, 8200, ("SlidingWindowChillMask", (3000, 2000)), (8100,)),
]


# The same kernel at head dim 64 (rows of 128 bytes: one slab of a tile per wave, transposed operands of the two
# 16-row halves at addresses of their own), on grids of at least 1024 workgroups; chunkwise masks from chunks of 320 rows on
DKDV_REGS_CASES_64 = [
    ("causal", torch.bfloat16, 4, 16, 16, 4096, ("CausalChillMask", ()), None),
    ("causal-gqa-lens-f16", torch.float16, 8, 16, 8, 4096, ("CausalChillMask", ()), (4096, 4000, 33, 2049, 4096, 1, 3111, 4095)),
    ("full-gqa-ragged", torch.bfloat16, 4, 32, 16, 4100, ("FullChillMask", ()), None),
    ("prefix-lm-gqa-ragged-lens-f16", torch.float16, 2, 64, 32, 4111, ("PrefixLMChillMask", (77,)), (4001, 4111)),
    ("long-prefix-lm", torch.bfloat16, 1, 32, 32, 8192, ("PrefixLMChillMask", (1024,)), None),
    ("chunkwise-512x1-f16", torch.float16, 2, 32, 16, 8192, ("ChunkwiseChillMask", (512, 1)), (8000, 8192)),
    ("sliding-4096+100", torch.bfloat16, 2, 32, 32, 8192, ("SlidingWindowChillMask", (4096, 100)), None),
    ("full-T1024", torch.bfloat16, 16, 16, 16, 1024, ("FullChillMask", ()), None),
    ("full-256-workgroups", torch.bfloat16, 1, 16, 16, 4096, ("FullChillMask", ()), None),
    ("causal-512-workgroups-T8192-gqa", torch.bfloat16, 1, 32, 16, 8192, ("CausalChillMask", ()), (8100,)),
    ("causal-T3500-gqa-f16", torch.float16, 10, 16, 8, 3500, ("CausalChillMask", ()), None),
]


# Banded masks whose rows see 1024 keys and more take the forward's 8-wave shape with its generated loop at head dim 128
# (narrower ones keep the 4-wave shape): runs of predicate-free tiles with masked tiles before and after them, waves of one
# workgroup whose runs differ, chunk sizes that are no multiple of a tile, a band wider than the sequence
WIDE_BAND_FWD_CASES = [
    ("sliding-1024+0", torch.bfloat16, 2, 4, 4, 4096, ("SlidingWindowChillMask", (1024, 0)), None, (256, 8)),
    ("sliding-700+700-ragged-lens-f16", torch.float16, 2, 4, 2, 4133, ("SlidingWindowChillMask", (700, 700)), (4133, 2500), (256, 8)),
    ("sliding-5000+0-wider-than-T", torch.bfloat16, 1, 8, 8, 3000, ("SlidingWindowChillMask", (5000, 0)), None, (256, 8)),
    ("chunkwise-1000x1-f16", torch.float16, 1, 8, 8, 4096, ("ChunkwiseChillMask", (1000, 1)), None, (256, 8)),
    ("chunkwise-512x1-gqa-lens", torch.bfloat16, 2, 8, 2, 4096, ("ChunkwiseChillMask", (512, 1)), (4000, 1111), (256, 8)),
    ("sliding-1000+22-narrow", torch.bfloat16, 1, 8, 8, 4096, ("SlidingWindowChillMask", (1000, 22)), None, (128, 4)),
    ("chunkwise-256x2-narrow-f16", torch.float16, 1, 8, 8, 4096, ("ChunkwiseChillMask", (256, 2)), None, (128, 4)),
]


@pytest.mark.parametrize("case", WIDE_BAND_FWD_CASES, ids=lambda c: c[0])
def test_forward_of_wide_bands_takes_the_long_loop(case):
    """O and LSE2 (chill_fwd.py:215-330 is what they must equal) and the gradients behind them on banded masks either
    side of the width from which the forward takes the shape of the masks that are not banded (route asserted)."""
    _, dtype, B, H, Hkv, T, m, lens, route = case
    D = 128
    mask = make_mask(m)
    cfg = tile_config(mask, D, dtype, _lib.PASS_FWD, seq_len=T, batch_heads=B * H)
    assert (cfg["rows"], cfg["waves"]) == route, f"served by {cfg}"
    torch.manual_seed(stable_seed(case[0]))
    q, k, v = (make_qkv((B, h, T, D), dtype, False).requires_grad_() for h in (H, Hkv, Hkv))
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    dout = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    out, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens_t, return_lse=True)
    out.backward(dout)
    qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
    ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens_t)
    ref.backward(dout.float() * res_mask)
    check_close(out.detach() * res_mask, ref.detach(), dtype, OUT_TOL[dtype], D, "O")
    want_lse = orc.lse2_dense(m[0], m[1], q.detach(), k.detach(), lens_t)
    seen = torch.isfinite(want_lse)  # (rows at and behind lens see no key)
    torch.testing.assert_close(lse[seen].double(), want_lse[seen], atol=2e-2, rtol=1e-3)
    for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
        check_close(got, want, dtype, GRAD_TOL[dtype], D, name)


def _random_long_cases(n, seed):
    """Seeded draws of (head dim, dtype, B, H, H_kv, T, mask, lens) among the shapes the launchers send to the kernels of long
    sequences: most grids above the thresholds of the register-resident kernels, some below; ragged lengths; every mask
    family with arguments either side of the widths and chunk sizes that change the route."""
    import random

    rng = random.Random(seed)
    cases = []
    for i in range(n):
        D = rng.choice([64, 128, 128])
        dtype = rng.choice([torch.bfloat16, torch.float16])
        T = rng.choice([4096, 4100, 5000, 6143, 8192, 8200, 9000, rng.randint(4096, 9500)])
        m = rng.choice([
            ("CausalChillMask", ()), ("FullChillMask", ()),
            ("PrefixLMChillMask", (rng.choice([1, 77, 1024, 3000, 5000]),)),
            ("SlidingWindowChillMask", (rng.choice([1023, 2048, 4096, 5000]), rng.choice([0, 0, 100, 2000]))),
            ("SlidingWindowChillMask", (rng.choice([0, 64, 500]), rng.choice([0, 64, 300]))),
            ("ChunkwiseChillMask", (rng.choice([64, 128, 320, 512, 1024]), rng.choice([0, 1, 3]))),
            ("ChunkwiseChillMask", (rng.choice([96, 100, 333, 1000]), rng.choice([0, 2]))),
            ("ChunkwiseChillMask", (rng.choice([512, 2048]), rng.choice([1, 2])))])
        group = rng.choice([1, 1, 2, 4])
        need = (512 if D == 128 else 1024) * 256 // T + 1  # B * H_kv from which dK/dV takes its register-resident kernel
        if rng.random() < 0.25:
            need = max(1, need // 4)
        B = rng.choice([1, 2, 4])
        Hkv = max(1, -(-need // B))
        H = Hkv * group
        if B * H * T * D * 2 > 400e6:
            H = max(group, int(400e6 / (B * T * D * 2)) // group * group)
            Hkv = H // group
        lens = None
        if rng.random() < 0.4:
            lens = tuple(rng.choice([T, T - 1, rng.randint(1, T), rng.randint(T // 2, T)]) for _ in range(B))
        cases.append((f"{i}-D{D}-{str(dtype)[6:]}-B{B}-H{H}/{Hkv}-T{T}-{m[0][:-9]}{list(m[1])}", D, dtype, B, H, Hkv, T, m, lens))
    return cases


# Grids of more workgroups than CUs that the chip still holds at once (two or three workgroups of four waves per CU):
# the kernels take every second pass over an XCD's CUs in reverse order.  Totals that are no multiple of 8 or 32, a last
# pass that is not full, GQA, lens.
RESIDENT_GRID_CASES = [
    ("resident-dq-330", 128, torch.bfloat16, 1, 10, 5, 4200, ("CausalChillMask", ()), None),
    ("resident-dq-480-f16", 128, torch.float16, 3, 5, 5, 4096, ("PrefixLMChillMask", (700,)), (4096, 4000, 2000)),
    ("resident-d64-297", 64, torch.bfloat16, 1, 9, 3, 4100, ("CausalChillMask", ()), (4001,)),
    ("resident-d64-dkdv-650-f16", 64, torch.float16, 2, 10, 5, 4100, ("CausalChillMask", ()), None),
    ("resident-d64-512", 64, torch.bfloat16, 1, 16, 16, 4096, ("SlidingWindowChillMask", (2000, 100)), None),
]


@pytest.mark.parametrize("case", _random_long_cases(32, 20240607) + RESIDENT_GRID_CASES, ids=lambda c: c[0])
def test_random_long_sequences(case):
    """Forward and backward against the dense reference (chill_fwd.py:215-330, chill_bwd_dq.py:300-394,
    chill_bwd_dkdv.py:347-508 are what they must equal) on seeded random draws of long shapes."""
    _, D, dtype, B, H, Hkv, T, m, lens = case
    mask = make_mask(m)
    torch.manual_seed(stable_seed(case[0]))
    q, k, v = (make_qkv((B, h, T, D), dtype, False).requires_grad_() for h in (H, Hkv, Hkv))
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    dout = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    out = ca.chill_attention(q, k, v, mask=mask, lens=lens_t)
    out.backward(dout)
    qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
    ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens_t)
    ref.backward(dout.float() * res_mask)
    check_close(out.detach() * res_mask, ref.detach(), dtype, OUT_TOL[dtype], D, "O")
    for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
        check_close(got, want, dtype, GRAD_TOL[dtype], D, name)
    if lens is not None:
        for b, n in enumerate(lens):
            assert (k.grad[b, :, n:] == 0).all() and (v.grad[b, :, n:] == 0).all() and (q.grad[b, :, n:] == 0).all()


@pytest.mark.parametrize("case", [c + (128,) for c in DKDV_REGS_CASES] + [c + (64,) for c in DKDV_REGS_CASES_64],
                         ids=lambda c: f"{c[0]}-D{c[-1]}")
def test_dkdv_with_resident_keys_and_generated_loop(case):
    """The dK/dV kernel that keeps K in registers and runs its predicate-free tiles in a generated loop (and, from 8192
    keys on, the dQ kernel that does the same with Q and dO), on shapes the launcher routes to them (asserted from the
    tile table): heads of a GQA group one after the other, lens, sequence
    lengths that leave a ragged last tile, the first tiles of a key block under the mask (run by the ordinary code).
    Same bar as the other backward tests (chill_bwd_dkdv.py:347-508 is what it must equal)."""
    _, dtype, B, H, Hkv, T, m, lens, D = case
    mask = make_mask(m)
    cfg = tile_config(mask, D, dtype, _lib.PASS_DKDV, seq_len=T, batch_heads=B * Hkv)
    assert (cfg["rows"], cfg["waves"], cfg["streamed"]) == (256, 4, 32), f"served by {cfg}"
    # (dQ has such a kernel too, for sequences from 4097 keys on, full masks from 2048)
    cfg = tile_config(mask, D, dtype, _lib.PASS_DQ, seq_len=T, batch_heads=B * H)
    banded = m[0] in ("ChunkwiseChillMask", "SlidingWindowChillMask")
    dq_regs = (not banded and D == 128 and T >= (2048 if m[0] == "FullChillMask" else 4097) and B * H * -(-T // 256) >= 512)
    assert ((cfg["rows"], cfg["waves"], cfg["streamed"]) == (256, 4, 32)) == dq_regs, f"dQ served by {cfg}"
    torch.manual_seed(stable_seed(case[0]))
    q, k, v = (make_qkv((B, h, T, D), dtype, False).requires_grad_() for h in (H, Hkv, Hkv))
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    dout = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    out = ca.chill_attention(q, k, v, mask=mask, lens=lens_t)
    out.backward(dout)
    qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
    ref, res_mask = orc.reference_naive(m[0], m[1], qf, kf, vf, lens_t)
    ref.backward(dout.float() * res_mask)
    check_close(out.detach() * res_mask, ref.detach(), dtype, OUT_TOL[dtype], D, "O")
    for name, got, want in (("dv", v.grad, vf.grad), ("dk", k.grad, kf.grad), ("dq", q.grad, qf.grad)):
        check_close(got, want, dtype, GRAD_TOL[dtype], D, name)
    # rows at and behind lens get no gradient
    if lens is not None:
        for b, n in enumerate(lens):
            assert (k.grad[b, :, n:] == 0).all() and (v.grad[b, :, n:] == 0).all()


def test_rows_without_keys():
    """A query whose keys are all masked (possible with lens cutting a window that only looks ahead)."""
    m = ("SlidingWindowChillMask", (0, 0))
    B, H, T, D = 1, 1, 64, 32
    q, k, v = (torch.randn(B, H, T, D, device=DEV) for _ in range(3))
    o, lse = ca.chill_attention(q, k, v, mask=make_mask(m), return_lse=True)
    torch.testing.assert_close(o, v, atol=1e-6, rtol=1e-6)  # each row sees only itself
    expected = (q * k).sum(-1) * D ** -0.5 * math.log2(math.e)
    torch.testing.assert_close(lse, expected, atol=1e-4, rtol=1e-5)


def test_strided_views_run_without_copy_and_match():
    """[B, T, H, D] storage viewed as [B, H, T, D] (unit inner stride) is consumed in place."""
    mask = ca.CausalChillMask()
    B, H, T, D = 2, 4, 300, 64
    base = [torch.randn(B, T, H, D, device=DEV, dtype=torch.bfloat16) for _ in range(3)]
    q, k, v = (x.transpose(1, 2) for x in base)
    assert not q.is_contiguous()
    out = ca.chill_attention(q, k, v, mask=mask)
    out_c = ca.chill_attention(q.contiguous(), k.contiguous(), v.contiguous(), mask=mask)
    assert torch.equal(out, out_c)
    # slices with a storage offset and a padded row pitch
    big = torch.randn(B, H, T, 2 * D, device=DEV, dtype=torch.bfloat16)
    qs, ks, vs = big[..., :D], big[..., D:], big[..., :D]
    out_s = ca.chill_attention(qs, ks, vs, mask=mask)
    assert torch.equal(out_s, ca.chill_attention(qs.contiguous(), ks.contiguous(), vs.contiguous(), mask=mask))


def test_gradients_through_strided_and_fp32_dout():
    mask = ca.PrefixLMChillMask(20)
    B, H, T, D = 2, 2, 130, 32
    q, k, v = (torch.randn(B, T, H, D, device=DEV, dtype=torch.float16).transpose(1, 2).requires_grad_() for _ in range(3))
    out = ca.chill_attention(q, k, v, mask=mask)
    dout = torch.randn(B, H, T, D, device=DEV, dtype=torch.float32)
    out.backward(dout)  # fp32 upstream gradient, as the reference's test passes it
    qf, kf, vf = (x.detach().float().clone().requires_grad_() for x in (q, k, v))
    ref, _ = orc.reference_naive("PrefixLMChillMask", (20,), qf, kf, vf, None)
    ref.backward(dout)
    for got, want in ((q.grad, qf.grad), (k.grad, kf.grad), (v.grad, vf.grad)):
        torch.testing.assert_close(got, want.half(), atol=5e-3, rtol=1e-3)


@pytest.mark.parametrize("D", [128, 64])
def test_register_resident_backward_on_strided_views(D):
    """The long-sequence backward kernels (K, or at head dim 128 Q and dO, in registers; tile pointers that the generated
    loops move on by a row stride) on [B, T, H, D] storage viewed as [B, H, T, D], a GQA group, and an upstream gradient
    with a padded row pitch: bit for bit what the same launch gives on contiguous copies."""
    mask = ca.CausalChillMask()
    B, H, Hkv, T = (2, 16, 8, 8192) if D == 128 else (2, 32, 16, 8192)  # (head dim 64: on grids of 1024 workgroups)
    dtype = torch.bfloat16
    for pss, cfg_heads in ((_lib.PASS_DKDV, B * Hkv), (_lib.PASS_DQ, B * H)):
        cfg = tile_config(mask, D, dtype, pss, seq_len=T, batch_heads=cfg_heads)
        assert ((cfg["rows"], cfg["waves"], cfg["streamed"]) == (256, 4, 32)) == (D == 128 or pss == _lib.PASS_DKDV), f"served by {cfg}"
    torch.manual_seed(11)
    q = torch.randn(B, T, H, D, device=DEV, dtype=dtype).transpose(1, 2).requires_grad_()
    k, v = (torch.randn(B, T, Hkv, D, device=DEV, dtype=dtype).transpose(1, 2).requires_grad_() for _ in range(2))
    dout = torch.randn(B, H, T, 2 * D, device=DEV, dtype=dtype)[..., D:]
    assert not q.is_contiguous() and not dout.is_contiguous()
    ca.chill_attention(q, k, v, mask=mask).backward(dout)
    qc, kc, vc = (x.detach().contiguous().requires_grad_() for x in (q, k, v))
    ca.chill_attention(qc, kc, vc, mask=mask).backward(dout.contiguous())
    for name, got, want in (("dq", q.grad, qc.grad), ("dk", k.grad, kc.grad), ("dv", v.grad, vc.grad)):
        assert torch.equal(got, want), name


def test_mask_args_are_runtime_values():
    """Instances of one mask class share one registered op; their arguments reach the kernel at run time."""
    q, k, v = (torch.randn(1, 2, 256, 64, device=DEV, dtype=torch.float16) for _ in range(3))
    a = ca.chill_attention(q, k, v, mask=ca.SlidingWindowChillMask(5, 1))
    b = ca.chill_attention(q, k, v, mask=ca.SlidingWindowChillMask(50, 20))
    ra, _ = orc.reference_naive("SlidingWindowChillMask", (5, 1), q.float(), k.float(), v.float())
    rb, _ = orc.reference_naive("SlidingWindowChillMask", (50, 20), q.float(), k.float(), v.float())
    torch.testing.assert_close(a, ra.half(), atol=1e-2, rtol=1e-3)
    torch.testing.assert_close(b, rb.half(), atol=1e-2, rtol=1e-3)
    assert hasattr(torch.ops.chill_attention, "forwardSlidingWindowChillMask")
    assert hasattr(torch.ops.chill_attention, "backwardSlidingWindowChillMask")


def test_opcheck_and_compile():
    mask = ca.CausalChillMask()
    ca.register_chill_mask(mask)
    q, k, v = (torch.randn(1, 2, 64, 32, device=DEV, dtype=torch.float32, requires_grad=True) for _ in range(3))
    torch.library.opcheck(
        torch.ops.chill_attention.forwardCausalChillMask.default,
        (q, k, v, None, [], 0.17, True, False, "ieee", False),
        test_utils=("test_schema", "test_faketensor", "test_autograd_registration"),
    )
    fn = torch.compile(lambda a, b, c: ca.chill_attention(a, b, c, mask=mask), fullgraph=True)
    out = fn(q, k, v)
    torch.testing.assert_close(out, ca.chill_attention(q, k, v, mask=mask))
    out.sum().backward()
    assert q.grad is not None and torch.isfinite(q.grad).all()


@pytest.mark.parametrize("m", [MASK_INSTANCES[1], MASK_INSTANCES[2]], ids=mask_id)
def test_hip_graph_replays(m):
    """Forward + backward captured once in a HIP graph: every replay, with new contents in the
    static inputs and eager work and synchronisations in between, equals the eager result.  (The
    library allocates nothing, keeps no state and launches only on the caller's stream.)"""
    mask = make_mask(m)
    B, H, Hkv, T, D = 2, 4, 2, 300, 128
    q, k, v = (torch.randn(B, h, T, D, device=DEV, dtype=torch.bfloat16, requires_grad=True) for h in (H, Hkv, Hkv))
    do = torch.randn(B, H, T, D, device=DEV, dtype=torch.bfloat16)
    lens = torch.tensor([T, 77], dtype=torch.int32, device=DEV)

    def step():
        out = ca.chill_attention(q, k, v, mask=mask, lens=lens)
        grads = torch.autograd.grad(out, (q, k, v), do)
        return (out,) + grads

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step()
    for replay in range(4):
        with torch.no_grad():
            for t in (q, k, v, do):
                t.copy_(torch.randn_like(t) * (1.0 + replay))
            lens.copy_(torch.tensor([T - 13 * replay, 77 + 50 * replay], dtype=torch.int32))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in static_out]
        want = step()
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w), f"replay {replay}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("D", [16, 64, 128, 256])
def test_delta_kernel(D, dtype):
    """chill_bwd_delta through the C ABI against the closed form rowsum(O * dO) in fp64 (utils.py:190),
    on strided inputs and a T that is not a multiple of the kernel's rows per block."""
    import ctypes

    from chill_attention import _lib

    B, H, T = 3, 5, 333
    o = torch.randn(B, T, H, D, device=DEV, dtype=dtype).transpose(1, 2)  # [B, H, T, D] view, strided
    do = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    delta = torch.full((B, H, T), float("nan"), device=DEV, dtype=torch.float32)
    to, tdo = _lib.tensor4(o), _lib.tensor4(do)
    _lib.check("chill_bwd_delta", _lib.lib.chill_bwd_delta(
        ctypes.byref(to), ctypes.byref(tdo), ctypes.c_void_p(delta.data_ptr()), _lib.strides3(delta),
        B, H, T, D, {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[dtype],
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    want = orc.delta(o.double().cpu().numpy(), do.double().cpu().numpy())
    # fp32 accumulation of D products of magnitude ~1
    np.testing.assert_allclose(delta.cpu().numpy(), want, atol=2e-5 * D, rtol=1e-5)


# One shape per dQ kernel: (id, dtype, D, B, H, Hkv, T, mask, lens, (rows, waves, streamed) of the dQ row)
DQ_DELTA_CASES = [
    ("eight-waves", torch.bfloat16, 128, 2, 8, 8, 4500, ("CausalChillMask", ()), (4500, 1000), (256, 8, 64)),
    ("four-waves-gqa-f16", torch.float16, 64, 2, 8, 2, 1100, ("PrefixLMChillMask", (100,)), None, (128, 4, 64)),
    ("four-waves-window", torch.bfloat16, 128, 1, 16, 16, 2100, ("SlidingWindowChillMask", (100, 30)), (1999,), (128, 4, 64)),
    ("registers-128", torch.bfloat16, 128, 1, 16, 8, 8200, ("CausalChillMask", ()), (8111,), (256, 4, 32)),
    ("registers-256-f16", torch.float16, 256, 1, 8, 8, 1030, ("FullChillMask", ()), (700,), (128, 4, 32)),
    ("split-f32-256", torch.float32, 256, 1, 4, 2, 530, ("CausalChillMask", ()), (333,), None),
    ("f32-64", torch.float32, 64, 4, 12, 12, 1500, ("ChunkwiseChillMask", (64, 2)), (1500, 65, 1, 777), (128, 4, 32)),
    ("small-launch", torch.bfloat16, 64, 1, 2, 1, 300, ("CausalChillMask", ()), (129,), (32, 4, 32)),
    ("small-launch-f32", torch.float32, 32, 1, 3, 3, 257, ("FullChillMask", ()), None, (32, 4, 32)),
]


@pytest.mark.parametrize("case", DQ_DELTA_CASES, ids=lambda c: c[0])
def test_dq_computes_delta_on_its_way(case):
    """chill_bwd_dq_delta (what the operator's backward launches before dK/dV) through the C ABI, on one shape per dQ
    kernel (route asserted from the tile table): the delta rows it leaves behind equal the closed form rowsum(O * dO)
    in fp64 (utils.py:190) on every row below lens[b] and are finite on every other row (the buffer starts as NaN),
    and its dQ equals what chill_bwd_dq computes from chill_bwd_delta's rows, up to the rounding of a sum of D
    products taken in another order."""
    import ctypes

    _, dtype, D, B, H, Hkv, T, m, lens, route = case
    mask = make_mask(m)
    if route is not None:
        cfg = tile_config(mask, D, dtype, _lib.PASS_DQ, seq_len=T, batch_heads=B * H)
        assert (cfg["rows"], cfg["waves"], cfg["streamed"]) == route, f"served by {cfg}"
    torch.manual_seed(stable_seed(case[0]))
    q, k, v = (make_qkv((B, h, T, D), dtype, False) for h in (H, Hkv, Hkv))
    do = torch.randn(B, T, H, D, device=DEV, dtype=dtype).transpose(1, 2)  # a strided view
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
    o, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens_t, return_lse=True)
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[dtype]
    desc = mask.descriptor()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    lens_p = (None, 0) if lens_t is None else (ctypes.c_void_p(lens_t.data_ptr()), lens_t.stride(0))
    t = {n: _lib.tensor4(x) for n, x in (("q", q), ("k", k), ("v", v), ("o", o), ("do", do))}
    r = lambda n: ctypes.byref(t[n])  # noqa: E731
    lse_p, s_lse = ctypes.c_void_p(lse.data_ptr()), _lib.strides3(lse)
    sm_scale = D ** -0.5
    L = _lib.lib
    # the two launches of the reference's structure
    delta = torch.empty(B, H, T, dtype=torch.float32, device=DEV)
    want = torch.full_like(q, float("nan"))
    tw = _lib.tensor4(want)
    _lib.check("chill_bwd_delta", L.chill_bwd_delta(r("o"), r("do"), ctypes.c_void_p(delta.data_ptr()), _lib.strides3(delta),
                                                    B, H, T, D, code, stream))
    _lib.check("chill_bwd_dq", L.chill_bwd_dq(r("q"), r("k"), r("v"), r("do"), ctypes.byref(tw), lse_p, s_lse,
                                              ctypes.c_void_p(delta.data_ptr()), _lib.strides3(delta), *lens_p, B, H, Hkv, T, D,
                                              code, sm_scale, ctypes.byref(desc), stream))
    # the fused one, into a buffer of NaNs
    delta2 = torch.full((B, H, T), float("nan"), dtype=torch.float32, device=DEV)
    got = torch.full_like(q, float("nan"))
    tg = _lib.tensor4(got)
    _lib.check("chill_bwd_dq_delta", L.chill_bwd_dq_delta(
        r("q"), r("k"), r("v"), r("o"), r("do"), ctypes.byref(tg), lse_p, s_lse, ctypes.c_void_p(delta2.data_ptr()),
        _lib.strides3(delta2), *lens_p, B, H, Hkv, T, D, code, sm_scale, ctypes.byref(desc), stream))
    torch.cuda.synchronize()
    assert torch.isfinite(delta2).all(), "a row of delta was left unwritten"
    closed = orc.delta(o.double().cpu().numpy(), do.double().cpu().numpy())
    for b in range(B):
        n = T if lens is None else lens[b]
        np.testing.assert_allclose(delta2[b, :, :n].cpu().numpy(), closed[b, :, :n], atol=2e-5 * D, rtol=1e-5)
    assert torch.isfinite(got).all()
    tol = {torch.float32: 1e-5, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]
    torch.testing.assert_close(got.float(), want.float(), atol=tol, rtol=tol)
    # and dK/dV from the rows the fused launch left behind equal dK/dV from chill_bwd_delta's rows to the same bar
    grads = []
    for rows in (delta, delta2):
        dk, dv = torch.full_like(k, float("nan")), torch.full_like(v, float("nan"))
        tdk, tdv = _lib.tensor4(dk), _lib.tensor4(dv)
        _lib.check("chill_bwd_dkdv", L.chill_bwd_dkdv(
            r("q"), r("k"), r("v"), r("do"), ctypes.byref(tdk), ctypes.byref(tdv), lse_p, s_lse,
            ctypes.c_void_p(rows.data_ptr()), _lib.strides3(rows), *lens_p, B, H, Hkv, T, D, code, sm_scale,
            ctypes.byref(desc), stream))
        grads.append((dk, dv))
    torch.cuda.synchronize()
    for a, b_ in zip(grads[0], grads[1]):
        assert torch.isfinite(b_).all()
        torch.testing.assert_close(b_.float(), a.float(), atol=tol, rtol=tol)


@pytest.mark.parametrize("T,D,dtype", [(70001, 64, torch.float16), (100003, 128, torch.bfloat16)])
def test_long_sequences(T, D, dtype):
    """Sequences far beyond the BASELINE sizes, of a length no tile divides (row offsets past 2^24 elements):
    O on row slices at the start, the middle and the end against dense fp32 attention over all keys, and the
    scale symmetry sum(dQ . Q) == sum(dK . K) of the gradients."""
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 2, T, D, device=DEV, dtype=dtype, requires_grad=True) for _ in range(3))
    do = torch.randn(1, 2, T, D, device=DEV, dtype=dtype)
    ki = torch.arange(T, device=DEV)[None, :]
    for mask, visible in (
        (ca.CausalChillMask(), lambda qi: ki <= qi),
        (ca.SlidingWindowChillMask(1000, 0), lambda qi: (ki <= qi) & (ki >= qi - 1000)),
        (ca.PrefixLMChillMask(5000), lambda qi: (ki < 5000) | (ki <= qi)),
    ):
        o = ca.chill_attention(q, k, v, mask=mask)
        dq, dk, dv = torch.autograd.grad(o, (q, k, v), do)
        assert all(torch.isfinite(x).all().item() for x in (o, dq, dk, dv)), mask
        for r0 in (0, T // 2 - 100, T - 300):
            qi = torch.arange(r0, r0 + 300, device=DEV)[:, None]
            scores = q[0, :, r0 : r0 + 300].float() @ k[0].float().transpose(-1, -2) * D**-0.5
            ref = torch.softmax(scores.masked_fill(~visible(qi), float("-inf")), -1) @ v[0].float()
            torch.testing.assert_close(o[0, :, r0 : r0 + 300].float(), ref, atol=1e-2, rtol=1e-2)
        a = (dq.double() * q.double()).sum().item()
        b = (dk.double() * k.double()).sum().item()
        assert abs(a - b) <= 2e-2 * max(abs(a), abs(b), 1.0), (mask, a, b)


def test_device_functors_equal_host():
    """The mask functors and tile decisions as executed ON THE GPU equal the host build bit for bit."""
    import ctypes

    from chill_attention import _lib

    for m in MASK_INSTANCES:
        mask = make_mask(m)
        desc = mask.descriptor()
        for n in (1, 33, 500, 1030):
            out = torch.empty(n, n, dtype=torch.uint8, device=DEV)
            _lib.check("chill_mask_eval_device", _lib.lib.chill_mask_eval_device(
                ctypes.byref(desc), n, ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
            assert torch.equal(out.bool().cpu(), mask.make_mask(n).cpu())
        for pass_id in (_lib.PASS_FWD, _lib.PASS_DQ, _lib.PASS_DKDV):
            for T, seq_len, tin, tout in ((1030, 1030, 32, 64), (1030, 517, 256, 64), (8192, 8192, 128, 64), (300, 1, 32, 32)):
                n_tiles = -(-T // tin)
                out = torch.empty(n_tiles, 4, dtype=torch.int32, device=DEV)
                _lib.check("chill_tile_ranges_device", _lib.lib.chill_tile_ranges_device(
                    ctypes.byref(desc), pass_id, T, seq_len, tin, tout, ctypes.c_void_p(out.data_ptr()),
                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
                assert torch.equal(out.cpu(), mask._calc_tile_ranges(T, tin, tout, pass_id, seq_len))
